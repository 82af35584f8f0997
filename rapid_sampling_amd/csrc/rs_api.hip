// MI355X (gfx950) token sampler: kernels and the C ABI of include/rapid_sampling.h.
//
// Steps per row (reference lines in /root/reference/sampling.cu):
//   1  x = sf((sf(l) - pen) * c), row max                         :208-227, :547-559
//   2  e = 2^(x - floor(max)) kept as bit patterns                :228-258
//   3  threshold = largest t with count{e>=t} >= top_k or mass{e>=t} >= top_p*D.
//      The reference finds it by a 4-way search on bit patterns with one pass
//      over the row per step (:261-329); here it is a radix selection on the
//      same bit patterns: a (count, mass) histogram over the top 10 bits, then
//      the few tokens of the boundary bin are gathered and resolved in LDS
//      (or, for huge bins, the next 7 bits are histogrammed, up to 4 levels).
//   4  counts and mass above / at the threshold                   :332-355
//   5  tie weight                                                 :365-371
//   6  inverse-CDF pick in index order                            :374-426
//   7  penalty decay + one-hot add, in place, from registers      :427-437
// Everything summed across tokens is an integer, so the result does not depend
// on how a row is cut up or in which order the pieces arrive.
//
// Ways through these steps (choose_path below; the results are the same integers on every one):
//
//   general kernel (sample_kernel, one launch): a row is worked by a CLUSTER of
//     G workgroups of 256 threads; each thread keeps R float4 (4R tokens) in
//     registers for the whole call, so the row is read from HBM exactly once.
//     The workgroups of a cluster exchange histograms, the slice maxima, the
//     boundary tokens and their kept masses through the row's record in the
//     workspace; what is exchanged carries its own completeness (counts that
//     add up, words that are non-zero once written), every wait is bounded.
//     Any top_k / top_p, penalties, any batch.
//
//   streaming path (stream_kernel + finish_kernel, two launches, no waits): for
//     calls of 2^17 tokens and more without penalties whose kept set is small
//     next to the row (top_k <= 1024, or a small nucleus), and, as a counting-only
//     variant, for calls that keep every token.  One pass over the logits leaves
//     per-row histograms and per-slice stashes of the largest tokens; one
//     workgroup per row finishes the row from them.  A row it cannot finish that
//     way it does alone, from the logits (finish_row_slow), and says so to the
//     caller's rs_policy, which routes the next calls of that kind.
//
//   wide path (stream_kernel counting only + wide_kernel + wide_finish_kernel,
//     three launches, no waits): kept sets of thousands of tokens (top_k > 1024,
//     flat distributions under top_p).  The second pass reads the rows again with
//     the boundary bin of the first known, counts the bin's next digit and sets
//     aside the tokens around the place where each slice expects the threshold.
//
//   row kernel (row_kernel, one launch, no workspace, no waits): the same kept sets
//     in rows of up to 65536 tokens when the call has rows enough to fill the GPU
//     with one workgroup of 1024 threads per row, the row in its registers.
//
//   one-launch path (fused_kernel): the streaming pass and the finish in one
//     grid, for calls with penalties that fit the device at once.
//
//   penalties at scale (stream_pen_kernel + finish_kernel + penalty_fix_kernel).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <new>

#include "rs_common.h"

// Workspace of rs_sample_static: one array per GPU inside the library's code object.  In host code
// this name is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) unsigned char scratch[RS_STATIC_SCRATCH_BYTES];

namespace rs {

// Launch-plus-one-read floor: same grid, each row read once (every load of a thread issued before
// the first use, non-temporal or plain), one int out.
template <int R, bool ONCE>
__global__ void __launch_bounds__(kThreads) floor_kernel(const float *logits, int64_t row_stride, int32_t *out,
                                                         int32_t V, uint32_t G)
{
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const uint32_t V4 = (uint32_t)V >> 2;
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + threadIdx.x;
    const uint4 *lg = reinterpret_cast<const uint4 *>(logits + (int64_t)row * row_stride);
    uint4 v[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint4 *q = lg + min(base4 + (uint32_t)(j * kThreads), V4 - 1);
        v[j] = ONCE ? load_once(q) : *q;
    }
    float m = -3.402823466e+38f;
#pragma unroll
    for (int j = 0; j < R; ++j)
        m = fmaxf(m, fmaxf(fmaxf(__uint_as_float(v[j].x), __uint_as_float(v[j].y)), fmaxf(__uint_as_float(v[j].z), __uint_as_float(v[j].w))));
    // one combine per workgroup: contended atomics on a few addresses would be timed instead of the read
    __shared__ uint32_t wmax[kWaves];
    const uint32_t k = wave_max_u32(fkey(m));
    if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(reinterpret_cast<uint32_t *>(out + row), max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
}

// Read-only kernels of other shapes, for the read bandwidth the device delivers: a workgroup goes through
// `per` pieces of kThreads * U float4 (U loads per thread in flight), either pieces that lie one after the
// other (a long contiguous stretch per workgroup), or grid-strided ones (a persistent grid that sweeps
// the rows front to back); XCD: workgroup b runs on XCD b mod 8, and the eight XCDs are given an eighth
// of the data each, so that what one XCD's L2 sees is one contiguous stretch.
template <int U, bool STRIDED, bool XCD>
__global__ void __launch_bounds__(kThreads) floor_sweep_kernel(const float *logits, int64_t row_stride, int32_t *out, int32_t V,
                                                               uint32_t pieces_per_row, uint32_t pieces, uint32_t per)
{
    const uint32_t V4 = (uint32_t)V >> 2;
    uint32_t wg = blockIdx.x, nwg = gridDim.x;
    uint32_t first = 0, span = pieces;                   // the stretch of pieces this workgroup's group of workgroups shares
    if (XCD) {
        const uint32_t x = blockIdx.x & 7u, share = (pieces + 7u) >> 3;
        first = x * share; span = min(share, pieces > first ? pieces - first : 0u);
        wg = blockIdx.x >> 3; nwg = (gridDim.x + 7u - x) >> 3;
    }
    float m = -3.402823466e+38f;
    for (uint32_t i = 0; i < per; ++i) {
        const uint32_t local = STRIDED ? wg + i * nwg : wg * per + i;
        if (local >= span) break;
        const uint32_t piece = first + local;
        const uint32_t row = piece / pieces_per_row, off4 = (piece - row * pieces_per_row) * (uint32_t)(kThreads * U) + threadIdx.x;
        const uint4 *lg = reinterpret_cast<const uint4 *>(logits + (int64_t)row * row_stride);
        uint4 v[U];
#pragma unroll
        for (int j = 0; j < U; ++j) v[j] = load_once(lg + min(off4 + (uint32_t)(j * kThreads), V4 - 1));
#pragma unroll
        for (int j = 0; j < U; ++j)
            m = fmaxf(m, fmaxf(fmaxf(__uint_as_float(v[j].x), __uint_as_float(v[j].y)), fmaxf(__uint_as_float(v[j].z), __uint_as_float(v[j].w))));
    }
    __shared__ uint32_t wmax[kWaves];
    const uint32_t k = wave_max_u32(fkey(m));
    if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = k;
    __syncthreads();
    if (threadIdx.x == 0) atomicMax(reinterpret_cast<uint32_t *>(out), max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
}

__global__ void philox_init_kernel(uint32_t *state, uint64_t seed, int32_t B)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    uint32_t *s = state + (size_t)b * 16;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0;
    s[0] = (uint32_t)seed; s[1] = (uint32_t)(seed >> 32);
    s[4] = (uint32_t)b;
}

// Clears device memory with plain stores (a recorded memset node misbehaves on graph replays).
__global__ void __launch_bounds__(256) fill_zero_kernel(uint4 *dst, size_t n16, unsigned char *tail, uint32_t ntail)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = make_uint4(0u, 0u, 0u, 0u);
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

__global__ void set_u32_kernel(uint32_t *dst, uint32_t value) { *dst = value; }

// What a call reads before it writes: the launch counters of the header (workgroups that have left,
// the eight ticket counters) and its row records.  The sticky error word, the place of the first wait
// that gave up, the wait limit and the words of the routing report (n_need, last_call) are left as
// they are: they are read across calls.
__global__ void __launch_bounds__(256) clear_records_kernel(WsHeader *hdr, uint4 *recs, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) recs[i] = make_uint4(0u, 0u, 0u, 0u);
    if (blockIdx.x == 0) {
        if (threadIdx.x == 0) hdr->finished = 0u;
        for (uint32_t i = threadIdx.x; i < 8u * 64u; i += 256u) hdr->ticket[i >> 6][i & 63u] = 0u;
    }
}

// Puts the sticky error word and the record of the first wait that gave up back to "none".
__global__ void clear_error_kernel(WsHeader *hdr)
{
    hdr->error = 0;
    hdr->gave_up[0] = 0u; hdr->gave_up[1] = 0u; hdr->gave_up[2] = 0u; hdr->gave_up[3] = 0u;
}

// ------------------------------------------------------------ host side ----

struct Geometry { int R; uint32_t G; };

// Tokens per thread (4R) and workgroups per row.  Large batches take long
// slices (few peers to meet, deep loads); a lone row is cut into a few dozen
// slices so that many CUs pull it from HBM at once.
static Geometry choose_geometry(int32_t B, int32_t V, bool pen, int force_r)
{
    const uint32_t V4 = (uint32_t)V / 4;
    const int maxR = pen ? 16 : 32;
    auto parts = [&](int R) { return (V4 + (uint32_t)(kThreads * R) - 1) / (uint32_t)(kThreads * R); };
    if (force_r) {
        // (a row of more than 64 workgroups only while the whole launch fits the GPU at once: one XCD
        // holds 64 workgroups of the largest variants, and a row's workgroups wait for each other)
        const int R = force_r;
        if ((R == 1 || R == 2 || R == 4 || R == 8 || R == 16 || R == 32) && R <= maxR && parts(R) <= (uint32_t)kMaxParts &&
            (parts(R) <= 64u || (uint64_t)B * parts(R) <= 512u))
            return {R, parts(R)};
    }
    // Measured on MI355X: a cluster works best with at most ~64 workgroups (each exchange costs
    // more the more peers poll), slices of 32 float4 per thread only pay for rows of a quarter
    // million tokens and more (the variant spills), and a call wants a few hundred workgroups in
    // flight.
    int minR = maxR;
    for (int R = 1; R <= maxR; R *= 2)
        if (parts(R) <= 64u) { minR = R; break; }
    const int topR = (V4 >= 65536u || minR > 16) ? maxR : (maxR < 16 ? maxR : 16);
    int pick = minR;
    if (B <= 16) {
        // a handful of rows: the shortest slices that keep the call within 256 workgroups (measured for 8 and
        // 16 rows of 32768 to 100256 tokens: 128-256 workgroups 20-24 us, 400-800 workgroups 25-37 us; one to
        // four rows are as fast with any length up to 8192 tokens)
        for (int R = minR; R <= topR; R *= 2) {
            pick = R;
            if ((uint64_t)B * parts(R) <= 256u) break;
        }
    } else {
        for (int R = topR; R >= minR; R /= 2)
            if ((uint64_t)B * parts(R) >= 512u) { pick = R; break; }
    }
    // A launch the device holds at once (256 CUs x the workgroups per CU of the variant, see
    // min_waves) draws no tickets, and tickets cost the first workgroups of a larger launch 10-15 us:
    // if a longer slice brings the launch within that, take it (measured on flat rows, 128-512 of
    // them: 13-24 % faster; when both lengths need tickets the shorter slice wins).
    auto resident = [&](int R) { const int data = (pen ? 8 : 4) * R; return 256u * (data <= 32 ? 4u : data <= 64 ? 3u : 2u); };
    if (parts(pick) > 1u && (uint64_t)B * parts(pick) > resident(pick))
        for (int R = pick * 2; R <= maxR; R *= 2)
            if ((uint64_t)B * parts(R) <= resident(R)) { pick = R; break; }
    return {pick, parts(pick)};
}


// Streaming geometry: workgroups of 256 threads.  Rows of up to 262144 tokens are cut into slices of
// 4096 tokens (4 float4 per thread) while all of the call's slices fit the device at once, else into
// slices of 8192 tokens while those do (256 CUs x 6 workgroups of either kernel = 1536), else into
// slices of 16384.  Measured over forty shapes of 4-13M tokens: a pass that is one wave of workgroups
// is 0.5-2.5 us per call faster with the shorter slices, and slower from the first workgroup beyond
// that.  Longer rows take slices of 16384 tokens (they would be cut into more slices than a
// finishing workgroup handles quickly) unless the call is only a few of them.
constexpr int kStreamNT = 256;
constexpr uint32_t kStreamSmallParts = 1536;
constexpr int32_t kMidMaxV = 262144;                          // rows up to here may be cut into slices of 8192 tokens whatever the call's size (wide_r)
constexpr uint64_t kFusedSmall = 1ull << 22;
static uint32_t stream_parts(int32_t V, int R) { return ((uint32_t)V / 4 + kStreamNT * R - 1) / (kStreamNT * R); }
// `pen`: the pass that also reads penalties exists for the long slices only
static int stream_r(int32_t B, int32_t V, bool pen = false)
{
    if (V > 262144) {
        // a few long rows: shorter slices while a row has at most 128 of them and the call at most 512
        // (measured at 524288 and 1048576 tokens: 1-3.7 us faster up to there, slower beyond)
        for (int R = 4; R <= 8 && !pen; R *= 2) {
            const uint32_t g = stream_parts(V, R);
            if (g <= 128u && (uint64_t)B * g <= 512u) return R;
        }
        return kStreamLongR;
    }
    if ((uint64_t)B * stream_parts(V, 4) <= kStreamSmallParts) return 4;
    if (!pen && (uint64_t)B * stream_parts(V, 8) <= kStreamSmallParts) return 8;
    return kStreamLongR;
}
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
struct StreamLayout { size_t hdr, cum, shist, stash, pens, end; };
// `with_pens`: room for every slice's note of its non-zero penalties behind the stashes (long slices only)
static StreamLayout stream_layout(size_t parts, size_t base, bool with_pens = false)
{
    StreamLayout l;
    l.hdr = align256(base);
    l.cum = align256(l.hdr + parts * sizeof(PartHdr));
    l.shist = align256(l.cum + parts * kSB * sizeof(uint32_t));
    l.stash = align256(l.shist + parts * kSB * sizeof(uint64_t));
    l.pens = align256(l.stash + parts * kStashCap * sizeof(uint64_t));
    l.end = with_pens ? align256(l.pens + parts * kPenCap * sizeof(uint64_t)) : l.pens;
    return l;
}
// Bytes of per-slice data a workspace for (B, V) sets aside: enough for the long slices of (B, V)
// itself and for the shorter slices of any call of at most B rows that takes them (the streaming
// path: at most kStreamSmallParts of them, of 4096 or of 8192 tokens; the one-launch path: calls of
// at most kFusedSmall tokens, fewer than kFusedSmall / 4096 + B slices), so that the size grows
// with B and with V and a workspace for the largest B and V serves every smaller call.
// (`least`: what every call needs; without it, also room for slices of 8192 tokens in rows of up to
// 262144, which the one-pass wide path and the counting-only pass take when they are given it: see wide_r)
static size_t stream_bytes(int32_t B, int32_t V, bool least)
{
    const size_t longs = stream_layout((size_t)B * stream_parts(V, kStreamLongR), sizeof(WsHeader), true).end;
    size_t small_parts = (size_t)B * stream_parts(V, 4);
    const size_t cap = (size_t)kStreamSmallParts + (size_t)B;
    static_assert(kStreamSmallParts >= kFusedSmall / 4096, "room for either kind of small call");
    if (small_parts > cap) small_parts = cap;
    const size_t shorts = stream_layout(small_parts, sizeof(WsHeader)).end;
    size_t bytes = longs > shorts ? longs : shorts;
    if (!least) {
        const size_t mids = stream_layout((size_t)B * stream_parts(V < kMidMaxV ? V : kMidMaxV, 8), sizeof(WsHeader)).end;
        if (mids > bytes) bytes = mids;
    }
    return bytes;
}
// Slice length of the one-pass wide path and of the counting-only pass (plain temperature sampling): as
// stream_r, but slices of 8192 tokens instead of 16384 in rows of up to 262144 tokens whenever the
// workspace has room for them (a workspace of rs_workspace_bytes has).  Measured, us per call, 16384- against
// 8192-token slices: one-pass wide path 128 x 100256 65 / 55, 128 x 262144 90 / 80, 256 x 131072 88 / 77,
// 512 x 100256 128 / 110, 512 x 262144 210 / 191; counting-only pass with its finish 512 x 100256 60 / 51,
// 512 x 131072 69 / 62, 512 x 262144 116 / 109.  (The pass with stashes gains nothing: 512 x 262144 110 / 117;
// the two-pass wide path's counting pass 256 x 262144 161 / 168, 512 x 131072 159 / 153.)
static int wide_r(int32_t B, int32_t V, size_t workspace_bytes)
{
    const int r = stream_r(B, V);
    if (r != kStreamLongR || V > kMidMaxV) return r;
    const size_t need = stream_layout((size_t)B * stream_parts(V, 8), sizeof(WsHeader)).end + (size_t)B * sizeof(RowCtl);
    return need <= (workspace_bytes & ~(size_t)255) ? 8 : r;
}

}  // namespace rs

// The caller's routing state (see rapid_sampling.h).  Calls are of one of three kinds -- 0 the streaming
// path with a bounding top_k, 1 without one (an attempt), 2 the wide path -- and of one of three size
// classes (tokens per call below 2^20, below 2^24, from 2^24 on), and every (kind, class) has a report
// word of its own in pinned host memory, "a row had to be done the slow way" as last reported by a call of
// that kind and class: workloads that share a policy (a lone flat row and a batch of peaked ones on one
// stream) do not flip each other's route.  word[2]: RS_ERR_DEVICE once a kernel gave up a wait.  away[]:
// calls routed away since the word was last seen set and the path tried; period[]: how many of them
// before it is tried again; good[]: calls in a row that found the word clear.
// A probe's word is "pending" (kWordPending, set by the host with the call) until the probe has run: calls of
// its kind issued in the meantime -- a caller that does not synchronise between calls issues many -- are
// probes too, not attempts that may have to do their rows the slow way; after kPendingMost of them the
// calls stay away as after a slow row, and the try after that is a probe again (which leaves the word set
// until it has run).
constexpr uint32_t kAwayFirst = 64u, kAwayMost = 1024u, kPendingMost = 64u;
constexpr int32_t kWordPending = 2;
constexpr int kKinds = 4, kClasses = 3;
struct rs_policy {
    int32_t *word;
    uint32_t away[kKinds * kClasses], period[kKinds * kClasses], good[kKinds * kClasses];
    uint32_t probed[kClasses];                           // calls without a bounding top_k of this class have been tried once (as a probe)
    uint32_t pending[kClasses];                          // calls issued since a probe of this class whose word is still pending
};
static inline int size_class(int32_t B, int32_t V)
{
    const uint64_t n = (uint64_t)B * (uint64_t)V;
    return n < (1ull << 20) ? 0 : n < (1ull << 24) ? 1 : 2;
}
static inline int policy_slot(int kind, int cls) { return kind * kClasses + cls; }
static inline int policy_word(int kind, int cls) { return 4 + policy_slot(kind, cls); }

namespace rs {

// The streaming path works when the kept set is small next to the row; a row for which it does
// not is done by its finishing workgroup alone, from the logits, which takes several times as long
// as the general kernel needs for a whole call of moderate size.  With a bounding top_k that takes
// unusual rows (ties of thousands of tokens); without one (nucleus sampling alone) it is simply a
// flat distribution, so such a call is an attempt.  The kernels report "a row went the slow way:
// yes/no" into a word of the caller's rs_policy, one word for calls with a bounding top_k and one
// for calls without, and this function looks at the word -- without waiting for anything; a stale
// value only delays the switch -- before it chooses the path of the next call.  While the word is
// set, calls of that kind go to the general kernel, and streaming is tried again after 64 of them;
// each try that fails doubles that number (up to 1024), and as many good streaming calls in a row
// as the last stay away lasted put it back to 64: a workload whose rows are always too flat pays
// for one slow call in a thousand, a rare slow row costs a handful of calls on the general kernel.
// Without a policy, calls with a bounding top_k always stream and calls without never do.
//
// Measured on MI355X, back to back: with a bounding top_k the streaming path beats the cluster
// kernel from 131072 tokens per call upwards (15-17 us for small calls against 16-31 us, 2-3
// times faster for large ones); below that the single launch wins by up to a microsecond.
enum { kPathCluster = 0, kPathStream = 1, kPathAttempt = 2, kPathFused = 3, kPathKeep = 4, kPathWide = 5, kPathProbe = 6, kPathWide1 = 7, kPathRow = 8 };
// The wide path (four launches, two reads of the logits) against the general kernel (one launch, its
// exchanges), measured on flat rows (U[0,1), top_p 0.9) and on N(0,1.5) with top_k 10000: the wide path
// wins from about 25 million tokens per call on in rows of 50304 tokens and more (96 x 262144: 88 against
// 102 us and 69 against 93; 256 x 100256: 92 against 96 and 75 against 88; 512 x 50304: 105 against 107
// and 86 against 97; 256 x 131072: 104 against 108 and 85 against 99; 32 x 1048576: 106 against 133;
// 512 x 262144: 280 against 395), loses below that (128 x 131072: 72 against 64 and 58 against 61) and
// in short rows (2048 x 32768: 225 against 193).
constexpr uint64_t kWideMin = 3ull << 23;
constexpr int32_t kWideMinV = 49152;
// The one-pass wide path (a sample of the row, then one pass over all of it) against the two-pass one,
// same rows: up to about 2^26 tokens per call the second pass of the two-pass path comes out of the
// Infinity Cache and the two are level (256 x 131072: 91 against 101 us and 87 against 84; 512 x 65536: 105
// against 106 and 103 against 91); from there on the one pass wins (256 x 262144: 134 against 154 and 123
// against 129; 512 x 262144: 228 against 290 and 211 against 231; 128 x 1048576: 233 against 263 and 192
// against 226).
constexpr uint64_t kWide1Min = 1ull << 26;
// In rows of up to 262144 tokens the one-pass wide path works on slices of 8192 tokens (wide_r), which
// moves its crossover with the general kernel down to about 12 million tokens per call (128 x 100256: 55
// against 65 us; 128 x 131072: 60 against 66; 128 x 151936: 64 against 78; 64 x 262144: 62 against 65;
// below: 64 x 131072 48 against 38, 32 x 262144 50 against 40) and puts it ahead of the two-pass path
// everywhere above (256 x 131072: 77 against 94; 512 x 262144: 191 against 266).
constexpr uint64_t kWide1MinMid = 12000000ull;
constexpr uint64_t kPenStreamMin = 1ull << 23;
// The row kernel (one workgroup per row, the row in its registers, one launch; rows of up to 65536 tokens, no
// penalties) against what else there is for kept sets the stashes cannot hold, same rows, us per call:
//   rows x tokens   general/wide  row kernel        rows x tokens   general/wide  row kernel
//    64 x  8192       19 / 15      18 / 14           96 x 50304       30 / 28      31 / 32
//   256 x  8192       22 / 18      18 / 15          128 x 50304       39 / 36      32 / 32
//   384 x  8192       24 / 19      32 / 25          256 x 50304       62 / 58      33 / 34
//   256 x 16384       27 / 27      21 / 20          384 x 50304       81 / 77      62 / 63
//   512 x 16384       32 / 33      39 / 36          512 x 50304      103 / 85      65 / 66
//    96 x 32768       25 / 24      26 / 24         1024 x 50304      171 / 146    128 / 131
//   256 x 32768       38 / 36      27 / 26         2048 x 50304      343 / 336    252 / 258
//   384 x 32768       45 / 43      49 / 45          128 x 65536       38 / 36      37 / 39
//   512 x 32768       58 / 55      52 / 47          256 x 65536       65 / 61      41 / 44
//  2048 x 32768      193 / 185    197 / 181        1024 x 65536      186 / 184    159 / 167
// Its time is that of one row (14 us for 8192 tokens, 20 for 16384, 26 for 32768, 33 for 50304, 42 for
// 65536) times the rounds of 256 rows the call makes: it wins whenever one round does (from 64 rows on in
// short rows, 128 in long ones), and in rows of 32768 tokens and more also over several rounds.
static bool row_suits(int32_t B, int32_t V)
{
    if (V > kRowMaxV || V < 8192) return false;
    if (B <= 256) return B >= (V < 32768 ? 64 : 128);
    if (V < 32768) return false;
    return B >= 512 || V >= 40000;                            // 257 to 511 rows: two rounds pay off in long rows only
}
// Plain temperature sampling (top_k = V, top_p = 1: every live token is kept) has no kept set to
// stash, but the streaming pass's bins alone say which slice holds the target: one pass at
// bandwidth that only counts, plus a second look at one slice per row, beats the general kernel's
// three exchanges for rows of 32768 tokens and more at every size measured from 131072 tokens per
// call on (13.5 against 16.0 us for one row of 262144, 107 against 280 us for 128 rows of 1048576,
// 70 against 84 us for 1024 rows of 32768); many short rows (2048 of 4096: 74 against 51 us) are
// better off with the general kernel, which does such a row in one workgroup without exchanges.

// Slice length of the one-launch path (float4 groups per thread), 0 when the call does not suit it.
// Its workgroups hold their compute units until their row is finished, so a call pays twice once it
// has more workgroups than the GPU holds at a time (256 CUs x 3, x 2 for the longest slices with
// penalties: registers): the shortest slice that keeps the call within that is taken.  Calls of up
// to kFusedSmall tokens may use any of the three lengths (the workspace has room for their short
// slices), larger ones the long slices only.  `any_size` (forced by the caller): longest slices
// whatever the number of workgroups.
static int fused_r(int32_t B, int32_t V, bool pen, bool any_size)
{
    const bool small_call = (uint64_t)B * (uint64_t)V <= kFusedSmall && V <= 262144;
    const int choices[3] = {4, 8, 16};
    for (int i = small_call ? 0 : 2; i < 3; ++i) {
        const int R = choices[i];
        const uint32_t parts = stream_parts(V, R);
        if (parts < 2u || parts > (uint32_t)kMaxParts) continue;
        const uint64_t resident = 256u * (R == 16 && pen ? 2u : 3u);
        if ((uint64_t)B * parts <= resident || (any_size && i == 2)) return R;
    }
    if (any_size && small_call && stream_parts(V, 4) >= 2u) return 4;
    return 0;
}

static int choose_path(int32_t B, int32_t V, int32_t top_k, float top_p, bool pen, const rs_options *opt)
{
    const bool bounded = top_k <= kStreamK;
    const int force = opt ? opt->path : RS_PATH_AUTO;
    if (force == RS_PATH_FUSED) return fused_r(B, V, pen, true) ? kPathFused : kPathCluster;
    // The one-launch path by default: calls with penalties whose kept set is bounded by top_k (the
    // general kernel, the only other way with penalties, spends most of its time in exchanges).
    if (force == RS_PATH_AUTO && pen && bounded && fused_r(B, V, pen, false)) return kPathFused;
    // Larger calls with penalties: the streaming pass with a pass over the penalties behind it, from
    // kPenStreamMin tokens on (measured crossover with the general kernel), long slices only.
    rs_policy *pol = opt ? opt->policy : nullptr;
    const int cls = size_class(B, V);
    // after a call of this kind with a slow row: the general kernel for a while, then another try
    bool retry = false;                                       // routed_away() let this call through after a stay away
    bool pending = false;                                     // a probe of this class has been issued and has not run yet
    auto routed_away = [&](int kind) {
        if (!pol) return false;
        const int slot = policy_slot(kind, cls);
        volatile int32_t *word = pol->word + policy_word(kind, cls);
        if (*word == kWordPending) {
            if (++pol->pending[cls] <= kPendingMost) { pending = true; return false; }
            *word = 1;                                        // no word of the probe yet: away for now, the retry is a probe again
        }
        if (*word == 0) {
            if (pol->period[slot] > kAwayFirst && ++pol->good[slot] >= pol->period[slot]) pol->period[slot] = kAwayFirst;
            pol->away[slot] = 0;
            return false;
        }
        pol->good[slot] = 0;
        if (++pol->away[slot] <= pol->period[slot]) return true;
        pol->away[slot] = 0;                                  // this call streams again; a failure sets the word anew
        pol->period[slot] = min(pol->period[slot] * 2u, kAwayMost);
        retry = true;
        return false;
    };
    if (pen && bounded && stream_r(B, V, true) == kStreamLongR && stream_parts(V, kStreamLongR) >= 2u) {
        if (force == RS_PATH_STREAM || force == RS_PATH_ATTEMPT) return kPathStream;
        if (force == RS_PATH_AUTO && (uint64_t)B * (uint64_t)V >= kPenStreamMin && !routed_away(0)) return kPathStream;
    }
    if (pen) return kPathCluster;
    if (force == RS_PATH_CLUSTER) return kPathCluster;
    const bool keep_all = top_k == V && !(top_p < 1.0f);
    if (keep_all && (force == RS_PATH_STREAM || force == RS_PATH_ATTEMPT)) return kPathKeep;
    if (force == RS_PATH_STREAM) return bounded ? kPathStream : kPathCluster;
    if (force == RS_PATH_ATTEMPT) return bounded ? kPathStream : kPathAttempt;
    if (force == RS_PATH_WIDE) return keep_all ? kPathKeep : kPathWide;
    if (force == RS_PATH_WIDE1) return keep_all ? kPathKeep : kPathWide1;
    if (force == RS_PATH_ROW) return V <= kRowMaxV ? kPathRow : kPathCluster;
    // Small calls: rows of fewer than 8192 tokens are one or two workgroups of the general kernel each, with
    // few or no exchanges (8.5 us for a row of 256 tokens); from 8192 tokens per row on the streaming
    // path's two launches are faster whatever the batch (one row of 8192 to 100256 tokens: 13.6-14.7
    // against 16.1-17.9 us, 16 rows: 14.5-15.8 against 16.8-21.3; measured per call between events).
    if ((uint64_t)B * (uint64_t)V < (1ull << 17) && V < 8192) return kPathCluster;
    if (keep_all && V >= 32768) return kPathKeep;              // shorter rows: one workgroup of the general kernel does a row in one go
    // kept sets the stashes cannot hold: the wide path from kWideMin tokens on, unless its rows have been
    // going the slow way (slices that are no fair samples of their rows, ties of thousands of tokens)
    // (short rows in calls of many: the row kernel; else the one-pass wide path first; when its rows have been going the slow way -- samples that are no fair
    // picture of their rows -- the two-pass one, which counts everything; then the general kernel)
    auto wide_or_general = [&]() {
        const uint64_t tokens = (uint64_t)B * (uint64_t)V;
        if (row_suits(B, V)) return (int)kPathRow;
        if (tokens >= (V <= kMidMaxV ? kWide1MinMid : kWide1Min) && V >= kWideMinV && !routed_away(2)) return (int)kPathWide1;
        if (tokens >= kWideMin && V >= kWideMinV && !routed_away(3)) return (int)kPathWide;
        return (int)kPathCluster;
    };
    if (!bounded && !(top_p < 1.0f)) return wide_or_general(); // a top_k of thousands and no nucleus: more than the stashes hold
    if (!pol) return bounded ? kPathStream : wide_or_general();
    if (!routed_away(bounded ? 0 : 1)) {
        if (bounded) return kPathStream;
        // Whether the streaming path suits a workload without a bounding top_k is found out by a PROBE: the
        // first call of that kind on a policy, and every call that tries again after a stay away, takes
        // the wide path -- whose time does not depend on the kept set -- and its finishing workgroups report
        // whether the rows' kept sets would have fitted the stashes.  An attempt that fails costs a pass
        // of one workgroup over the row (hundreds of microseconds); a probe that says no costs nothing extra.
        // (a retry leaves the word set while its probe is under way: the calls behind it stay away)
        if (!pol->probed[cls] || retry || pending) {
            if (!pending && !retry) { pol->word[policy_word(1, cls)] = kWordPending; pol->pending[cls] = 0u; }
            pol->probed[cls] = 1u;
            return kPathProbe;
        }
        return kPathAttempt;
    }
    // (also with a bounding top_k whose rows have long lists all the same -- flat rows with a top_k of a
    // thousand: 128 x 100256 55 us on the one-pass wide path against 63 on the general kernel)
    return wide_or_general();
}

static hipError_t fill_zero(void *dst, size_t bytes, hipStream_t st)
{
    const size_t n16 = bytes / 16;
    const uint32_t blocks = (uint32_t)(n16 / 256 < 1 ? 1 : n16 / 256 > 2048 ? 2048 : n16 / 256);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, st, (uint4 *)dst, n16,
                       (unsigned char *)dst + n16 * 16, (uint32_t)(bytes - n16 * 16));
    return hipGetLastError();
}

}  // namespace rs

using namespace rs;

extern "C" {

int rs_version(void) { return 415; }

const char *rs_error_string(int code)
{
    switch (code) {
    case RS_OK:              return "ok";
    case RS_ERR_VOCAB:       return "Vocabulary size must be multiple of 4, and no larger than 1048576";
    case RS_ERR_BATCH:       return "B and T must be positive";
    case RS_ERR_TEMPERATURE: return "Temperature outside range, expect [0.001, 1000]";
    case RS_ERR_NULL:        return "a required pointer is NULL";
    case RS_ERR_WORKSPACE:   return "workspace too small or not 256-byte aligned";
    case RS_ERR_ALIGN:       return "rows of logits/penalties must be 16-byte aligned";
    case RS_ERR_ARG:         return "top_k/top_p not normalised: need 1 <= top_k <= V and 0 < top_p <= 1";
    case RS_ERR_LAUNCH:      return "HIP launch failed";
    case RS_ERR_DEVICE:      return "a workgroup gave up waiting for its peers";
    case RS_ERR_SCRATCH:     return "the call needs a larger workspace than the static scratch of rs_sample_static (RS_STATIC_SCRATCH_BYTES)";
    case RS_ERR_UNSUPPORTED: return "the device is not a whole MI355X (256 compute units in 8 XCDs): the kernels' waits are only known to end on one";
    default:                 return "unknown error";
    }
}

int rs_normalize_args(double temperature, int64_t top_k, double top_p,
                      int64_t B, int64_t T, int64_t V,
                      float *log2e_inv_temp, int32_t *top_k_out, float *top_p_out)
{
    if (!log2e_inv_temp || !top_k_out || !top_p_out) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (!(B > 0 && T > 0)) return RS_ERR_BATCH;
    if (!(temperature >= 0.001 && temperature <= 1000)) return RS_ERR_TEMPERATURE;
    if (top_k <= 0 || top_k > V) top_k = V;
    if (top_p < 0 || top_p > 1) top_p = 1;
    if (top_p == 0) { top_k = 1; top_p = 1; }
    *log2e_inv_temp = (float)(1.4426950408889634074 / temperature);
    *top_k_out = (int32_t)top_k;
    *top_p_out = (float)top_p;
    return RS_OK;
}

int rs_workspace_bytes(int32_t B, int32_t V, size_t *bytes)
{
    if (!bytes) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    *bytes = stream_bytes(B, V, false) + (size_t)B * sizeof(RowCtl);
    return RS_OK;
}

int rs_workspace_init(void *ws, size_t bytes, void *stream)
{
    if (!ws) return RS_ERR_NULL;
    if (bytes < sizeof(WsHeader) || ((uintptr_t)ws & 255)) return RS_ERR_WORKSPACE;
    return fill_zero(ws, bytes, (hipStream_t)stream) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

int rs_workspace_set_wait_limit(void *ws, uint32_t milliseconds, void *stream)
{
    if (!ws) return RS_ERR_NULL;
    if ((uintptr_t)ws & 255) return RS_ERR_WORKSPACE;
    if (milliseconds >= 40000u) return RS_ERR_ARG;
    const uint32_t ticks = (uint32_t)((uint64_t)milliseconds * 100000ull >> 10);      // 100 MHz wall clock
    hipLaunchKernelGGL(set_u32_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, &((WsHeader *)ws)->spin_ticks, ticks);
    return hipGetLastError() == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

int rs_workspace_status(const void *ws, int32_t *status, void *stream)
{
    if (!ws || !status) return RS_ERR_NULL;
    int32_t e = 0;
    const WsHeader *h = (const WsHeader *)ws;
    if (hipMemcpyAsync(&e, &h->error, sizeof e, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess) return RS_ERR_LAUNCH;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return RS_ERR_LAUNCH;
    *status = e;
    return RS_OK;
}

int rs_workspace_where(const void *ws, uint32_t where[4], void *stream)
{
    if (!ws || !where) return RS_ERR_NULL;
    const WsHeader *h = (const WsHeader *)ws;
    if (hipMemcpyAsync(where, h->gave_up, sizeof h->gave_up, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess)
        return RS_ERR_LAUNCH;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return RS_ERR_LAUNCH;
    return RS_OK;
}

int rs_policy_create(rs_policy **out)
{
    if (!out) return RS_ERR_NULL;
    *out = nullptr;
    rs_policy *pol = new (std::nothrow) rs_policy;
    if (!pol) return RS_ERR_LAUNCH;
    pol->word = nullptr;
    for (int i = 0; i < kKinds * kClasses; ++i) { pol->away[i] = 0; pol->good[i] = 0; pol->period[i] = kAwayFirst; }
    for (int i = 0; i < kClasses; ++i) { pol->probed[i] = 0; pol->pending[i] = 0; }
    if (hipHostMalloc((void **)&pol->word, 64, hipHostMallocDefault) != hipSuccess || !pol->word) {
        delete pol;
        return RS_ERR_LAUNCH;
    }
    for (int i = 0; i < 16; ++i) pol->word[i] = 0;
    *out = pol;
    return RS_OK;
}

void rs_policy_destroy(rs_policy *pol)
{
    if (!pol) return;
    if (pol->word) (void)hipHostFree(pol->word);
    delete pol;
}

int rs_policy_state(const rs_policy *pol, int32_t *state)
{
    if (!pol || !state) return RS_ERR_NULL;
    const volatile int32_t *w = pol->word;
    auto set = [&](int kind, int cls) { const int32_t x = w[policy_word(kind, cls)]; return x != 0 && x != kWordPending; };
    auto any = [&](int kind) { return set(kind, 0) || set(kind, 1) || set(kind, 2); };
    *state = (any(1) ? 1 : 0) | (any(0) ? 2 : 0) | (any(2) ? 4 : 0) | (any(3) ? 8 : 0);
    return RS_OK;
}

int rs_policy_error(rs_policy *pol, int32_t *error, int32_t clear)
{
    if (!pol || !error) return RS_ERR_NULL;
    volatile int32_t *w = pol->word;
    *error = w[2];
    if (clear) w[2] = 0;
    return RS_OK;
}

int rs_philox_init(void *state, uint64_t seed, int32_t B, void *stream)
{
    if (!state) return RS_ERR_NULL;
    if (B <= 0) return RS_ERR_BATCH;
    hipLaunchKernelGGL(philox_init_kernel, dim3((B + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       (uint32_t *)state, seed, B);
    return hipGetLastError() == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

int rs_sample(const float *logits, int64_t row_stride, float *penalties, int32_t *out,
              void *rng_state, const float *injected_u, int32_t B, int32_t V,
              float presence, float repetition, float decay,
              float log2e_inv_temp, int32_t top_k, float top_p,
              void *workspace, size_t workspace_bytes,
              rs_row_diag *diag, uint32_t *e_bits, void *stream)
{
    return rs_sample_ex(logits, RS_DTYPE_F32, row_stride, penalties, out, rng_state, injected_u, B, V, presence,
                        repetition, decay, log2e_inv_temp, top_k, top_p, workspace, workspace_bytes, diag, e_bits,
                        nullptr, stream);
}

int rs_sample_dtype(const void *logits, int32_t logits_dtype, int64_t row_stride, float *penalties, int32_t *out,
                    void *rng_state, const float *injected_u, int32_t B, int32_t V,
                    float presence, float repetition, float decay,
                    float log2e_inv_temp, int32_t top_k, float top_p,
                    void *workspace, size_t workspace_bytes,
                    rs_row_diag *diag, uint32_t *e_bits, void *stream)
{
    return rs_sample_ex(logits, logits_dtype, row_stride, penalties, out, rng_state, injected_u, B, V, presence,
                        repetition, decay, log2e_inv_temp, top_k, top_p, workspace, workspace_bytes, diag, e_bits,
                        nullptr, stream);
}

// The argument checks of a sampling call; nothing is launched before they pass.
static int check_call(const void *logits, int32_t logits_dtype, int64_t row_stride, const float *penalties, const int32_t *out,
                      const void *rng_state, const float *injected_u, int32_t B, int32_t V,
                      float log2e_inv_temp, int32_t top_k, float top_p, const uint32_t *e_bits, const rs_options *opt)
{
    if (!logits || !out || (!rng_state && !injected_u)) return RS_ERR_NULL;
    if (logits_dtype != RS_DTYPE_F32 && logits_dtype != RS_DTYPE_BF16 && logits_dtype != RS_DTYPE_F16) return RS_ERR_ARG;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    if (!(top_k >= 1 && top_k <= V) || !(top_p > 0.0f && top_p <= 1.0f) || !(log2e_inv_temp > 0.0f)) return RS_ERR_ARG;
    if (opt && (opt->path < RS_PATH_AUTO || opt->path > RS_PATH_ROW || opt->slice_r < 0)) return RS_ERR_ARG;
    if (((uintptr_t)logits & (logits_dtype == RS_DTYPE_F32 ? 15 : 7)) || (B > 1 && (row_stride & 3)) || ((uintptr_t)penalties & 15) || ((uintptr_t)e_bits & 15))
        return RS_ERR_ALIGN;
    return RS_OK;
}

// Compute units of the current device, looked up once per device (a host-side table lookup, no GPU
// work).  Every path with waits -- the general kernel, the one-launch kernel -- sizes its launches and
// its tickets for a whole MI355X: 256 compute units in 8 XCDs.  A partitioned device (compute-partition
// modes) or a CU-masked process holds fewer workgroups than those launches assume, rows could starve
// and every such call would end in a 2 s bounded wait: such a device is refused instead.
static int device_is_whole()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cus[kMaxDevices];            // 0 = not looked up yet
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return RS_ERR_LAUNCH;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (!n) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return RS_ERR_LAUNCH;
        cus[dev].store(n, std::memory_order_relaxed);
    }
    return n == 256 ? RS_OK : RS_ERR_UNSUPPORTED;
}

int rs_sample_ex(const void *logits, int32_t logits_dtype, int64_t row_stride, float *penalties, int32_t *out,
                 void *rng_state, const float *injected_u, int32_t B, int32_t V,
                 float presence, float repetition, float decay,
                 float log2e_inv_temp, int32_t top_k, float top_p,
                 void *workspace, size_t workspace_bytes,
                 rs_row_diag *diag, uint32_t *e_bits, const rs_options *opt, void *stream)
{
    if (!workspace) return RS_ERR_NULL;
    const int bad = check_call(logits, logits_dtype, row_stride, penalties, out, rng_state, injected_u, B, V, log2e_inv_temp,
                               top_k, top_p, e_bits, opt);
    if (bad != RS_OK) return bad;
    // (what the call cannot do without; rs_workspace_bytes asks for room for the shorter slices of wide_r on top)
    const size_t need = stream_bytes(B, V, true) + (size_t)B * sizeof(RowCtl);
    if (workspace_bytes < need || ((uintptr_t)workspace & 255)) return RS_ERR_WORKSPACE;
    const int whole = device_is_whole();
    if (whole != RS_OK) return whole;

    const bool pen = penalties != nullptr;
    const Geometry g = choose_geometry(B, V, pen, opt ? opt->slice_r : 0);
    Params p;
    p.logits = logits; p.dtype = logits_dtype; p.penalties = penalties; p.out = out;
    p.rng = (uint32_t *)rng_state; p.inj_u = injected_u; p.diag = diag; p.e_bits = e_bits;
    p.hdr = (WsHeader *)workspace;
    p.ctl_end = (RowCtl *)((char *)workspace + (workspace_bytes & ~(size_t)255));
    p.row_stride = row_stride; p.B = B; p.V = V; p.G = g.G;
    p.presence = presence; p.repetition = repetition; p.decay = decay; p.c = log2e_inv_temp;
    p.top_k = top_k; p.top_p = top_p;
    p.stash_k = (uint32_t)top_k; p.report = 0; p.attempt = 0;
    p.host_words = opt && opt->policy ? opt->policy->word : nullptr;
    p.defer_pen = 0; p.probe = 0;
    // Long lists on the streaming path are worth a report where another kernel does such rows faster: the
    // general kernel in calls of fewer than 2^24 tokens, the row kernel (whose time does not depend on the
    // kept set) in every call it suits
    p.tell_lists = ((uint64_t)B * (uint64_t)V < (1ull << 24) || row_suits(B, V)) ? 1u : 0u;
    dim3 grid((uint32_t)B * g.G);
    const int path = choose_path(B, V, top_k, top_p, pen, opt);
    if (path == kPathRow) return launch_row(logits_dtype, (uint32_t)B, (hipStream_t)stream, p) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
    if (path != kPathCluster) {
        const int sr = path == kPathFused ? fused_r(B, V, pen, opt && opt->path == RS_PATH_FUSED)
                     : (path == kPathWide1 || path == kPathKeep) ? wide_r(B, V, workspace_bytes) : stream_r(B, V, pen);
        StreamView v;
        v.G = stream_parts(V, sr);
        const bool pen_stream = pen && path == kPathStream;                  // long slices: their layout has room for the notes
        const StreamLayout l = stream_layout((size_t)B * v.G, sizeof(WsHeader), pen_stream);
        // (rs_workspace_bytes sets aside room for every slice length chosen above; checked all the same: a
        // layout that ran into the rows' records would be written out of bounds by thousands of workgroups)
        if (l.end + (size_t)B * sizeof(RowCtl) > (workspace_bytes & ~(size_t)255)) return RS_ERR_WORKSPACE;
        char *w = (char *)workspace;
        v.hdr = (PartHdr *)(w + l.hdr); v.stash = (uint64_t *)(w + l.stash); v.cum = (uint32_t *)(w + l.cum);
        v.shist = (uint64_t *)(w + l.shist);
        v.pens = pen_stream ? (uint64_t *)(w + l.pens) : nullptr;
        // without a bounding top_k the stashes are sized as for top_k = kStreamK: enough for a nucleus
        // of up to about a thousand tokens
        const uint32_t kk = min((uint32_t)top_k, (uint32_t)kStreamK);
        p.stash_k = min(kk, max(32u, 8u * kk / v.G));            // eight times a slice's share of the row's top_k
        hipStream_t st = (hipStream_t)stream;
        // The finishing workgroup's list: twice what a well-behaved row needs (its top_k tokens and
        // a boundary bin, or every stash whole), as a power of two; a row that needs more is handed
        // on.  Kept small where it can be: the list is LDS, and LDS decides how many rows finish at once.
        const uint32_t whole = v.G * (p.stash_k + 64u);            // every stash whole; of no use beyond kFinCap
        const uint32_t est = 2u * max(kk + 512u, whole <= (uint32_t)kFinCap ? whole : 0u);
        v.list_cap = 2048u;
        while (v.list_cap < est && v.list_cap < (uint32_t)kFinCap) v.list_cap *= 2u;
        // The one-launch path keeps its list, 2048 tokens, in static LDS it holds anyway, and never more
        // (a row that needs more falls back inside the kernel).  Its workgroups wait for each other, and
        // the hardware binds workgroup b to XCD b mod 8 before it starts: towards the end of a launch
        // the workgroups still to start may all belong to one XCD, and if that XCD's compute units were
        // all held by waiting workgroups of the row they belong to, nobody would ever move.  So a row
        // (at most 64 slices here) must be smaller than what ONE XCD holds: 32 CUs x 2 or 3 workgroups
        // with static LDS alone -- with a 64 KB list in dynamic LDS it was 32 x 1, and rows of 33 and
        // more slices could, rarely, starve until their waits gave up.
        if (path == kPathFused) v.list_cap = 2048u;
        const int kind = path == kPathAttempt || path == kPathProbe ? 1 : path == kPathWide1 ? 2 : path == kPathWide ? 3 : 0;
        p.report = path == kPathKeep ? 0u : (uint32_t)policy_word(kind, size_class(B, V));
        p.attempt = path == kPathAttempt ? 1u : 0u;
        p.probe = path == kPathProbe ? 1u : 0u;
        if (path == kPathKeep) { p.stash_k = 1u; v.list_cap = 2048u; }
        if (path == kPathWide || path == kPathProbe) {
            // the list holds the tokens of ONE sub-bin of the boundary bin: 1/128 of it for a smooth distribution
            p.stash_k = 1u; v.list_cap = 4096u;
            return launch_wide(sr, logits_dtype, (uint32_t)B, (size_t)v.list_cap * sizeof(uint64_t), st, p, v) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
        }
        if (path == kPathWide1) {
            p.stash_k = 1u; v.list_cap = 4096u;
            return launch_wide1(sr, logits_dtype, (uint32_t)B, (size_t)v.list_cap * sizeof(uint64_t), st, p, v) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
        }
        const size_t dyn = (size_t)v.list_cap * sizeof(uint64_t);
        if (path == kPathFused)
            return launch_fused(sr, pen, (uint32_t)B, st, p, v) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
        if (pen) {
            // penalties: read and rewritten (decayed) by the streaming pass, the sampled token's patched by the
            // finishing workgroup; slices the pass deferred are rewritten by a fix-up kernel at the end
            // a finite decay keeps +0.0 at +0.0, which is what lets the pass skip the groups that hold nothing
            p.defer_pen = (decay - decay == 0.0f) ? 2 : 1;
            if (launch_stream_pen((uint32_t)B, dyn, st, p, v) != hipSuccess) return RS_ERR_LAUNCH;
            return launch_penalty_fix(st, p, v) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
        }
        return launch_stream(sr, logits_dtype, path == kPathKeep, (uint32_t)B, dyn, st, p, v) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
    }
    return launch_sample(pen, g.R, grid, (hipStream_t)stream, p) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

// The static workspace of the current device: the array's address on that device, looked up once per
// device (every GPU holds its own copy of the array at its own address).
static int static_base(void **out)
{
    constexpr int kMaxDevices = 64;
    static std::atomic<void *> base[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return RS_ERR_LAUNCH;
    void *ws = base[dev].load(std::memory_order_acquire);
    if (!ws) {
        if (hipGetSymbolAddress(&ws, HIP_SYMBOL(scratch)) != hipSuccess || !ws) return RS_ERR_LAUNCH;
        base[dev].store(ws, std::memory_order_release);
    }
    *out = ws;
    return RS_OK;
}

int rs_static_prepare(void)
{
    void *ws = nullptr;
    return static_base(&ws);
}

void *rs_static_workspace(void)
{
    void *ws = nullptr;
    return static_base(&ws) == RS_OK ? ws : nullptr;
}

int rs_static_status(int32_t *status, uint32_t where[4], int32_t clear, void *stream)
{
    if (!status) return RS_ERR_NULL;
    void *ws = nullptr;
    const int rc = static_base(&ws);
    if (rc != RS_OK) return rc;
    int r = rs_workspace_status(ws, status, stream);
    if (r == RS_OK && where) r = rs_workspace_where(ws, where, stream);
    if (r == RS_OK && clear && *status != RS_OK) {
        hipLaunchKernelGGL(clear_error_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, (WsHeader *)ws);
        if (hipGetLastError() != hipSuccess) return RS_ERR_LAUNCH;
    }
    return r;
}

int rs_sample_static(const void *logits, int32_t logits_dtype, int64_t row_stride, float *penalties, int32_t *out,
                     void *rng_state, const float *injected_u, int32_t B, int32_t V,
                     float presence, float repetition, float decay,
                     float log2e_inv_temp, int32_t top_k, float top_p,
                     rs_row_diag *diag, uint32_t *e_bits, const rs_options *opt, void *stream)
{
    // everything that can refuse the call comes before the first launch
    const int bad = check_call(logits, logits_dtype, row_stride, penalties, out, rng_state, injected_u, B, V, log2e_inv_temp,
                               top_k, top_p, e_bits, opt);
    if (bad != RS_OK) return bad;
    const size_t need = stream_bytes(B, V, true) + (size_t)B * sizeof(RowCtl);  // what the call cannot do without
    if (need > (size_t)RS_STATIC_SCRATCH_BYTES) return RS_ERR_SCRATCH;
    const int whole = device_is_whole();
    if (whole != RS_OK) return whole;
    // the array of the CURRENT device is used, so the stream must belong to that device
    if (stream) {
        int cur = -1;
        hipDevice_t sdev = -1;
        if (hipGetDevice(&cur) != hipSuccess || hipStreamGetDevice((hipStream_t)stream, &sdev) != hipSuccess) return RS_ERR_LAUNCH;
        if ((int)sdev != cur) return RS_ERR_ARG;
    }
    void *ws = nullptr;
    const int rb = static_base(&ws);
    if (rb != RS_OK) return rb;
    // The array keeps what the last call left.  A call leaves it clean unless a wait gave up; the launch
    // counters and this call's row records are cleared all the same, by a kernel (not a memset node: the
    // call may be under capture), so that every call starts from zero whatever came before.  The sticky
    // error word stays (rs_static_status reads and clears it), and so do the words of the routing report.
    const size_t rec_bytes = (size_t)B * sizeof(RowCtl);
    char *recs = (char *)ws + (size_t)RS_STATIC_SCRATCH_BYTES - rec_bytes;
    const size_t n16 = rec_bytes / 16;
    const uint32_t blocks = (uint32_t)(n16 / 1024 < 1 ? 1 : n16 / 1024 > 1024 ? 1024 : n16 / 1024);
    hipLaunchKernelGGL(clear_records_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (WsHeader *)ws, (uint4 *)recs, n16);
    if (hipGetLastError() != hipSuccess) return RS_ERR_LAUNCH;
    return rs_sample_ex(logits, logits_dtype, row_stride, penalties, out, rng_state, injected_u, B, V, presence,
                        repetition, decay, log2e_inv_temp, top_k, top_p, ws, (size_t)RS_STATIC_SCRATCH_BYTES, diag,
                        e_bits, opt, stream);
}

int rs_floor_read(const float *logits, int64_t row_stride, int32_t *out, int32_t B, int32_t V, int32_t variant, void *stream)
{
    if (!logits || !out) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    if (variant < 0 || variant > 8) return RS_ERR_ARG;
    const uint32_t V4 = (uint32_t)V / 4;
    const bool once = (variant & 1) != 0;
    hipStream_t st = (hipStream_t)stream;
    if (variant >= 4) {
        // non-temporal loads throughout; pieces of kThreads * U float4
        auto sweep = [&](auto kernel, uint32_t U, uint32_t grid_or_0, uint32_t per_or_0) {
            const uint32_t ppr = (V4 + kThreads * U - 1) / (kThreads * U), pieces = (uint32_t)B * ppr;
            const uint32_t grid = grid_or_0 ? min(grid_or_0, pieces) : (pieces + per_or_0 - 1) / per_or_0;
            const uint32_t per = per_or_0 ? per_or_0 : (pieces + grid - 1) / grid + 1;
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, st, logits, row_stride, out, V, ppr, pieces, per);
        };
        switch (variant) {
        case 4: sweep(floor_sweep_kernel<4, true, false>, 4u, 2048u, 0u); break;     // persistent, 8 workgroups per CU, grid-strided, 4 loads in flight
        case 5: sweep(floor_sweep_kernel<4, true, true>, 4u, 2048u, 0u); break;      // the same, an eighth of the data per XCD
        case 6: sweep(floor_sweep_kernel<16, false, false>, 16u, 0u, 4u); break;     // 256 KiB per workgroup, contiguous, 16 loads in flight
        case 7: sweep(floor_sweep_kernel<8, true, true>, 8u, 1024u, 0u); break;      // persistent, 4 workgroups per CU, per XCD, 8 loads in flight
        default: sweep(floor_sweep_kernel<2, true, false>, 2u, 4096u, 0u); break;    // persistent, 16 workgroups per CU, 2 loads in flight
        }
        return hipGetLastError() == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
    }
#define RS_FLOOR(Rv) do { const uint32_t G = (V4 + kThreads * Rv - 1) / (kThreads * Rv); const dim3 grid((uint32_t)B * G);                          \
        if (once) hipLaunchKernelGGL((floor_kernel<Rv, true>), grid, dim3(kThreads), 0, st, logits, row_stride, out, V, G);                     \
        else hipLaunchKernelGGL((floor_kernel<Rv, false>), grid, dim3(kThreads), 0, st, logits, row_stride, out, V, G); } while (0)
    if (variant >= 2) {
        // the streaming pass's own geometry
        if (stream_r(B, V) == 4) RS_FLOOR(4); else if (stream_r(B, V) == 8) RS_FLOOR(8); else RS_FLOOR(kStreamLongR);
    } else {
        switch (choose_geometry(B, V, false, 0).R) {
        case 1:  RS_FLOOR(1); break;
        case 2:  RS_FLOOR(2); break;
        case 4:  RS_FLOOR(4); break;
        case 8:  RS_FLOOR(8); break;
        case 16: RS_FLOOR(16); break;
        default: RS_FLOOR(32); break;
        }
    }
#undef RS_FLOOR
    return hipGetLastError() == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

}  // extern "C"
