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
// Two ways through these steps:
//
//   cluster path (sample_kernel, one launch): a row is worked by a CLUSTER of
//     G workgroups of 256 threads; each thread keeps R float4 (4R tokens) in
//     registers for the whole call, so the row is read from HBM exactly once.
//     The workgroups of a cluster exchange histograms, the slice maxima, the
//     boundary tokens and their kept masses through the row's record in the
//     workspace; what is exchanged carries its own completeness (counts that
//     add up, words that are non-zero once written), every wait is bounded.
//     Any top_k / top_p, penalties, any batch.
//
//   streaming path (stream_kernel, finish_kernel, sample_list_kernel): for
//     calls of 2^17 tokens and more without penalties whose kept set is small
//     next to the row (top_k <= 1024, or a small nucleus).  No workgroup waits
//     for another: one pass over the logits leaves per-row histograms and
//     per-slice stashes of the largest tokens, a small kernel finishes each
//     row from them, and rows it cannot finish that way go through the
//     cluster kernel afterwards.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <new>

#include "rapid_sampling.h"
#include "rs_device.h"

// Workspace of rs_sample_static: one array per GPU inside the library's code object.  In host code
// this name is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) unsigned char scratch[RS_STATIC_SCRATCH_BYTES];

namespace rs {

constexpr int      kThreads   = 256;          // 4 waves, one per SIMD
constexpr int      kWaves     = kThreads / kWave;
constexpr int      kMaxParts  = 256;          // workgroups per row, at most
constexpr int      kNB        = 512;          // bins per histogram: level 1 uses 164, deeper levels 128
constexpr int      kLevels    = 4;            // 10 + 7 + 7 + 7 bits
constexpr int      kCap       = 1024;         // tokens of a boundary bin that are gathered
constexpr uint64_t kSpinLimit = 200000000ull; // 2 s of the 100 MHz wall clock

constexpr uint64_t kValid     = 1ull << 63;   // marks a written exchange word

struct alignas(256) WsHeader {
    uint32_t ticket;      // next logical workgroup id of the running launch
    uint32_t finished;    // workgroups that have left the running launch
    int32_t  error;       // sticky RS_ERR_DEVICE
    uint32_t n_need;      // rows the streaming pass handed to the cluster kernel
    uint32_t spin_ticks;  // bound of a wait in units of 1024 wall-clock ticks; 0 = the default (2 s)
    uint32_t pad[59];
};

// How long a workgroup waits for its peers before it gives up (wall-clock ticks).
__device__ __forceinline__ uint64_t spin_limit(const WsHeader *hdr)
{
    const uint32_t t = hdr->spin_ticks;
    return t ? (uint64_t)t << 10 : kSpinLimit;
}

// Per-row record.  Everything a call reads before writing it is zero when the
// call starts: the call itself re-zeroes what it used before it ends.  The
// records sit at the END of the workspace, row r at ctl_end[-1 - r], so that
// a row's record is at the same address whatever B and V a call has; the
// streaming path's per-slice data, which is written before it is read and
// never cleaned, grows from the front.  The two do not meet as long as the
// workspace is at least rs_workspace_bytes(largest B, largest V) of the calls
// that share it.
struct alignas(256) RowCtl {
    uint32_t done;        // workgroups finished with this row
    uint32_t cursor;      // fill of cand[]
    uint32_t index_p1;    // sampled token + 1, once known
    uint32_t pad[5];
    uint32_t mx[kMaxParts];     // per workgroup: fkey(max x of its slice), 0 = not yet written
    uint64_t A[2 * kMaxParts];  // per workgroup: a 124-bit mass as two words of 62 bits, each | kValid
    uint64_t cand[kCap];        // gathered tokens: bits << 32 | index
    uint64_t h[kLevels + 1][kNB];   // cluster histograms, packed (see kPackOne); one spare for the re-framed level 1
    uint64_t rowhist[kNB];          // streaming path: the row's bins by absolute octave (mod 128), summed over its slices
};

struct Params {
    const void  *logits;       // fp32, or bf16 / fp16 (dtype): converted exactly on load
    float       *penalties;
    int32_t     *out;
    uint32_t    *rng;          // 16 words per row, or null
    const float *inj_u;        // or null
    rs_row_diag *diag;         // or null
    uint32_t    *e_bits;       // or null
    WsHeader    *hdr;
    RowCtl      *ctl_end;      // one past the record of row 0; row r is ctl_end[-1 - r]
    uint32_t     stash_k;      // streaming pass: tokens a slice aims to stash (<= top_k)
    const uint32_t *need;      // null, or the list of rows this launch is for (hdr->n_need entries)
    int32_t      dtype;        // RS_DTYPE_* of the logits
    uint32_t     report;       // which of the two report words a streaming call writes: 0 top_k bounds the kept set, 1 not
    int32_t     *host_words;   // the caller's rs_policy: pinned host memory, [0], [1] routing reports, [2] error; or null
    int64_t      row_stride;
    int32_t      B, V;
    uint32_t     G;            // workgroups per row
    float        presence, repetition, decay, c;
    int32_t      top_k;
    float        top_p;
};

#define RS_AGENT __HIP_MEMORY_SCOPE_AGENT

// Everything workgroups exchange goes through relaxed device-scope atomics
// (they act at the level all XCDs share).  No exchange uses an arrival
// counter: completeness is visible in the data itself.
template <typename T> __device__ __forceinline__ T a_load(const T *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, RS_AGENT); }
template <typename T> __device__ __forceinline__ void a_store(T *p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, RS_AGENT); }
template <typename T> __device__ __forceinline__ void a_add(T *p, T v) { __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, RS_AGENT); }
__device__ __forceinline__ void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Hides a register from the optimiser for one use, so that work derived from
// the resident tokens is redone in each pass instead of being hoisted and kept
// in more registers per token.
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// ---- radix digits and histogram packing ----------------------------------
// The threshold is selected digit by digit on the bit pattern of e, largest e
// first.  Level 1 looks at bits [30:21]: index = bits >> 21 runs from 348
// (e = 2^-40) to 511 (e just below 2), 4 bins per octave aligned with the
// octaves, so every token of a bin has the same exponent (index >> 2).
// Levels 2..4 take 7 more bits each (shifts 14, 7, 0).  Histograms are stored
// by index (ascending in e); the scan walks them by digit = top - index.
constexpr uint32_t kTop1 = 511u;                      // largest index at level 1
constexpr uint32_t kBin0 = 348u;                      // smallest: e = 2^-40
constexpr uint32_t kTopN = 127u;                      // largest index of a deeper level
__device__ __forceinline__ uint32_t level_shift(uint32_t level) { return 21u - 7u * (level - 1u); }   // level >= 2

// A bin is one 64-bit word: count << 43 | sum of the tokens' 23 fraction bits.
// With the shared exponent ex the bin's exact mass is
// (sum + count * 2^23) << (ex - 87).  Counts stay below 2^21 and sums below
// 2^43 for any row of at most 2^20 tokens, so one atomic add carries both.
constexpr uint64_t kPackOne  = 1ull << 43;
constexpr uint64_t kPackMask = kPackOne - 1;
__device__ __forceinline__ uint32_t pack_count(uint64_t w) { return (uint32_t)(w >> 43); }
__device__ __forceinline__ u128 pack_mass(uint64_t w, uint32_t ex)
{
    return (u128)((w & kPackMask) + ((w >> 43) << 23)) << (ex - 87u);
}

// Bits of e in a frame `delta` octaves above the one they were computed in
// (delta <= 64): the exponent drops by delta; what falls below 2^-40 is dead
// (kept at or above 2^-41).
__device__ __forceinline__ uint32_t rebase_bits(uint32_t b, uint32_t delta)
{
    const uint32_t d = delta << 23;
    return max(b, d + kDeadBits) - d;
}

// Logits arrive as fp32 or, if the caller opted in, as bf16 or fp16.  Both widen to fp32
// exactly, so everything behind the load is the same arithmetic on the same values.
__device__ __forceinline__ const char *logits_row(const Params &p, uint32_t row)
{
    return static_cast<const char *>(p.logits) + (int64_t)row * p.row_stride * (p.dtype == RS_DTYPE_F32 ? 4 : 2);
}
__device__ __forceinline__ void widen4(uint2 h, int dtype, uint32_t *bits)
{
    if (dtype == RS_DTYPE_BF16) {
        bits[0] = h.x << 16; bits[1] = h.x & 0xFFFF0000u; bits[2] = h.y << 16; bits[3] = h.y & 0xFFFF0000u;
    } else {
        bits[0] = __float_as_uint((float)__builtin_bit_cast(_Float16, (uint16_t)(h.x & 0xFFFFu)));
        bits[1] = __float_as_uint((float)__builtin_bit_cast(_Float16, (uint16_t)(h.x >> 16)));
        bits[2] = __float_as_uint((float)__builtin_bit_cast(_Float16, (uint16_t)(h.y & 0xFFFFu)));
        bits[3] = __float_as_uint((float)__builtin_bit_cast(_Float16, (uint16_t)(h.y >> 16)));
    }
}
// group i4 (four tokens) of a row as floats, any dtype: for the rare re-reads
__device__ __forceinline__ float4 load_logits4(const char *rowp, uint32_t i4, int dtype)
{
    if (dtype == RS_DTYPE_F32) return reinterpret_cast<const float4 *>(rowp)[i4];
    uint32_t b[4];
    widen4(reinterpret_cast<const uint2 *>(rowp)[i4], dtype, b);
    return make_float4(__uint_as_float(b[0]), __uint_as_float(b[1]), __uint_as_float(b[2]), __uint_as_float(b[3]));
}

struct Found {               // result of a histogram scan (uniform over the workgroup)
    u128     mass_above;
    u128     local_above;    // level 1 only: mass of this workgroup's own tokens above the bin
    uint32_t bin;            // index of the first bin (largest e first) at which the kept set becomes sufficient
    uint32_t cnt_above;      // tokens in bins before it (plus the carried offset)
    uint32_t cnt_bin;        // tokens in it
    uint32_t pad;
};

constexpr int kRepC = 4;
struct Lds {
    u128     q128[kWaves * 2];
    u128     bc128[4];
    u128     wj[kWaves][32];
    u128     tj[32];
    u128     D, P;
    Found    found;
    uint64_t hm[kNB];        // this workgroup's histogram
    uint64_t hr[kNB * kRepC]; // level 1 while it is being counted: kRepC copies of each bin (lane l adds to copy
                             // l % kRepC), since lanes that add to one LDS address are served one after the other
                             // and rows often put most of their tokens into a few bins
    uint64_t g[kNB];         // the cluster's histogram
    uint64_t cand[kCap];
    uint64_t bc64[8];
    uint32_t u32[kWaves * 4];
    uint32_t bc32[8];
    uint32_t ctr;
    int      abort;
    int32_t *host_words;     // Params::host_words, for the code that gives up a wait
};

__device__ __forceinline__ uint32_t block_max_u32(Lds &s, uint32_t v, int lane, int wave)
{
    v = wave_max_u32(v);
    __syncthreads();
    if (lane == 0) s.u32[wave] = v;
    __syncthreads();
    uint32_t r = s.u32[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) r = s.u32[w] > r ? s.u32[w] : r;
    return r;
}

__device__ __forceinline__ uint32_t block_sum_u32(Lds &s, uint32_t v, int lane, int wave)
{
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) s.u32[wave] = v;
    __syncthreads();
    uint32_t r = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += s.u32[w];
    return r;
}

__device__ __forceinline__ u128 block_sum_u128(Lds &s, u128 v, int lane, int wave)
{
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) s.q128[wave] = v;
    __syncthreads();
    u128 r = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += s.q128[w];
    return r;
}

// two sums at once
__device__ __forceinline__ void block_sum2_u128(Lds &s, u128 &a, u128 &b, int lane, int wave)
{
    a = wave_sum(a); b = wave_sum(b);
    __syncthreads();
    if (lane == 0) { s.q128[wave * 2] = a; s.q128[wave * 2 + 1] = b; }
    __syncthreads();
    a = 0; b = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) { a += s.q128[w * 2]; b += s.q128[w * 2 + 1]; }
}

// A wait that ran out of time: the sticky error word of the workspace, the caller's pinned host
// word if there is one (readable without synchronising), and the flag that makes the workgroup leave.
struct Lds;
__device__ __forceinline__ void give_up(Lds &s, WsHeader *hdr);

// Bounded wait bookkeeping: thread 0 looks at the wall clock now and then; the
// verdict is read by everyone after a workgroup barrier, so it is uniform.
struct SpinGuard {
    uint64_t t0;
    uint32_t spins;
    __device__ __forceinline__ void start() { t0 = (uint64_t)wall_clock64(); spins = 0; }
    // call by every thread once per polling round, before the round's __syncthreads
    __device__ __forceinline__ void tick(Lds &s, WsHeader *hdr)
    {
        if (threadIdx.x == 0 && (++spins & 255u) == 0 && (uint64_t)wall_clock64() - t0 > spin_limit(hdr)) give_up(s, hdr);
    }
};

__device__ __forceinline__ void give_up(Lds &s, WsHeader *hdr)
{
    a_store(&hdr->error, (int32_t)RS_ERR_DEVICE);
    if (s.host_words) __hip_atomic_store(s.host_words + 2, (int32_t)RS_ERR_DEVICE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    s.abort = 1;
}

__device__ __forceinline__ void lds_hist_zero(Lds &s, int nb)
{
    for (int b = threadIdx.x; b < nb; b += kThreads) s.hm[b] = 0;
}
// one LDS atomic per token: count and fraction bits together
__device__ __forceinline__ void lds_hist_add(Lds &s, uint32_t bin, uint32_t b)
{
    atomicAdd(reinterpret_cast<unsigned long long *>(&s.hm[bin]), (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
}

// Re-zero this workgroup's share of a global histogram (the cluster splits the bins).
__device__ __forceinline__ void zero_slice(uint64_t *gh, uint32_t nb, uint32_t part, uint32_t G)
{
    const uint32_t lo = (uint32_t)(((uint64_t)nb * part) / G), hi = (uint32_t)(((uint64_t)nb * (part + 1)) / G);
    for (uint32_t b = lo + threadIdx.x; b < hi; b += kThreads) a_store(&gh[b], (uint64_t)0);
}

// Sum the workgroup histograms of a cluster: add mine (s.hm, kept) into the
// row's global bins with one 64-bit atomic per non-empty bin, then read the
// bins back until their counts add up to `expected` -- count and value of a
// contribution arrive in one word, so a complete count means complete data
// and no arrival counter is needed.  The totals end in s.g.  A cluster of one
// copies its own.  Returns false when the wait gave up.
__device__ __forceinline__ bool hist_combine(Lds &s, WsHeader *hdr, uint32_t G, uint64_t *gh, int nb, uint32_t expected,
                                             int lane, int wave)
{
    __syncthreads();
    if (G == 1) {
        for (int b = threadIdx.x; b < nb; b += kThreads) s.g[b] = s.hm[b];
        __syncthreads();
        return true;
    }
    for (int b = threadIdx.x; b < nb; b += kThreads) {
        const uint64_t v = s.hm[b];
        if (v) a_add(&gh[b], v);
    }
    SpinGuard guard;
    guard.start();
    for (;;) {
        uint32_t c = 0;
        for (int b = threadIdx.x; b < nb; b += kThreads) {
            const uint64_t w = a_load(&gh[b]);
            s.g[b] = w;
            c += pack_count(w);
        }
        guard.tick(s, hdr);
        const uint32_t total = block_sum_u32(s, c, lane, wave);
        if (total == expected) return true;
        if (s.abort) return false;
    }
}

// Level 1 of a cluster of several workgroups.  s.hm holds this slice's bins by
// absolute octave position; they are added to the row's (gh) and the row's are
// polled until complete, together with the slots of the slice maxima (thread t
// takes slot t).  Once all is there the row's frame M = floor(max) is known,
// and both histograms are stored in that frame: position c holds bin 348 + r,
// r = c - pos(M) mod 512; r >= 164 lies below 2^-40 of the frame, where
// tokens are dead: they were counted (the counts must add up) and are dropped.
// Indices below 348 of s.g and s.hm are left stale.  A slice's dead tokens
// sit one octave below its 41 live ones, so positions are shared safely while
// the slices' maxima lie within 86 octaves of each other.  Returns 0 on
// success, 1 when they do not (s.g and s.hm are then undefined), -1 when the
// wait gave up.
__device__ __forceinline__ int combine_level1(Lds &s, WsHeader *hdr, uint32_t G, uint64_t *gh, const uint32_t *slots,
                                              uint32_t expected, uint32_t &kmax_out, int lane, int wave)
{
    const int tid = threadIdx.x;
    __syncthreads();
    const uint64_t h0 = s.hm[tid], h1 = s.hm[tid + kThreads];
    if (h0) a_add(&gh[tid], h0);
    if (h1) a_add(&gh[tid + kThreads], h1);
    uint64_t g0, g1;
    uint32_t kmax, kmin;
    SpinGuard guard;
    guard.start();
    for (;;) {
        g0 = a_load(&gh[tid]); g1 = a_load(&gh[tid + kThreads]);
        uint32_t c = pack_count(g0) + pack_count(g1);
        uint32_t key = 0, nkey = 0;
        if ((uint32_t)tid < G) {
            key = a_load(&slots[tid]);                   // never 0 once written; a missing slot spoils the sum
            nkey = ~key;
            c += key == 0u ? 1u << 24 : 0u;
        }
        guard.tick(s, hdr);
        c = wave_sum(c); key = wave_max_u32(key); nkey = wave_max_u32(nkey);
        __syncthreads();
        if (lane == 0) { s.u32[wave] = c; s.u32[kWaves + wave] = key; s.u32[2 * kWaves + wave] = nkey; }
        __syncthreads();
        uint32_t total = 0;
        kmax = 0; kmin = 0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            total += s.u32[w]; kmax = max(kmax, s.u32[kWaves + w]); kmin = max(kmin, s.u32[2 * kWaves + w]);
        }
        if (total == expected) break;
        if (s.abort) return -1;
    }
    kmin = ~kmin;
    kmax_out = kmax;
    const float M = __builtin_floorf(fkey_inv(kmax));
    if (!(M - __builtin_floorf(fkey_inv(kmin)) < 87.0f)) return 1;
    const uint32_t m4 = (uint32_t)(int)(M - 128.0f * __builtin_floorf(M * 0.0078125f)) * 4u;
    const uint32_t r0 = ((uint32_t)tid + 160u - m4) & 511u, r1 = ((uint32_t)tid + kThreads + 160u - m4) & 511u;
    if (r0 < 164u) { s.g[kBin0 + r0] = g0; s.hm[kBin0 + r0] = h0; }
    if (r1 < 164u) { s.g[kBin0 + r1] = g1; s.hm[kBin0 + r1] = h1; }
    __syncthreads();
    return 0;
}

// Scan the level-1 histogram s.g from the top (index 511, largest e) down to
// index 348 (e = 2^-40) and find the first bin at which (count so far >=
// top_k) or (mass so far >= P).  The total mass of the histogram is the row
// total D, and P = ceil(top_p * D) is derived from it here.  The 164 bins fit
// one wave (lane l owns indices 511-3l, 510-3l, 509-3l), so the scan needs no
// LDS exchange; the exponent of bin idx is idx >> 2.  With LOCAL the wave also
// scans this workgroup's own histogram s.hm and returns its mass above the
// boundary bin in local_above.  With GIVEN_P the histogram is that of a
// subset of the row which is complete above some value: D and P are left alone.
template <bool LOCAL, bool GIVEN_P = false>
__device__ __forceinline__ Found hist_find_level1(Lds &s, uint64_t top_k, float top_p, int lane, int wave)
{
    if (wave == 0) {
        uint32_t c[3]; u128 m[3], hl[3];
        uint32_t cs = 0; u128 ms = 0, hs = 0;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int idx = (int)kTop1 - 3 * lane - i;
            const uint64_t w = idx >= (int)kBin0 ? s.g[idx] : 0ull;
            c[i] = pack_count(w);
            m[i] = w ? pack_mass(w, (uint32_t)idx >> 2) : (u128)0;
            cs += c[i]; ms += m[i];
            if (LOCAL) {
                const uint64_t h = idx >= (int)kBin0 ? s.hm[idx] : 0ull;
                hl[i] = h ? pack_mass(h, (uint32_t)idx >> 2) : (u128)0;
                hs += hl[i];
            }
        }
        const u128 mi = wave_inclusive_scan(ms);
        const uint32_t ci = wave_inclusive_scan(cs);
        u128 hrun = 0;
        if (LOCAL) hrun = wave_inclusive_scan(hs) - hs;
        u128 P;
        if (GIVEN_P) {
            // the histogram holds only part of the row: P stands as it is, and the scan may end
            // without the set becoming sufficient (bin 0 then)
            P = s.P;
            if (lane == 0) s.found.bin = 0;
        } else {
            const u128 D = lane63(mi);
            P = ceil_mul(top_p, D);
            if (lane == 0) { s.D = D; s.P = P; }
        }
        uint64_t rcnt = (uint64_t)ci - cs;               // count before my first bin
        u128 rm = mi - ms;                               // mass before my first bin
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const bool before = rcnt >= top_k || rm >= P;
            const uint64_t nc = rcnt + c[i];
            const u128 nm = rm + m[i];
            const bool after = nc >= top_k || nm >= P;
            if (!before && after) {
                s.found.bin = kTop1 - (uint32_t)(3 * lane + i);
                s.found.cnt_above = (uint32_t)rcnt; s.found.cnt_bin = c[i];
                s.found.mass_above = rm;
                s.found.local_above = hrun;
            }
            rcnt = nc; rm = nm;
            if (LOCAL) hrun += hl[i];
        }
    }
    __syncthreads();
    return s.found;
}

// A boundary bin with nothing above it holds the row's largest token.  Every token of the bin
// shares its exponent and none has a larger fraction, so a fraction sum of count times the largest
// token's fraction proves that all of them equal it: one tie, whose value is then known without
// looking at another digit.  `word` is the bin's packed count and fraction sum.
__device__ __forceinline__ bool bin_is_one_tie(uint64_t word, uint32_t bin, uint32_t emax_bits)
{
    return (emax_bits >> 21) == bin && (word & kPackMask) == (uint64_t)pack_count(word) * (uint64_t)(emax_bits & 0x7FFFFFu);
}

// The same for a 128-bin level (all tokens share the exponent ex): one wave,
// lane l owns indices 127-2l and 126-2l, no LDS exchange inside the scan.
__device__ __forceinline__ Found hist_find128(Lds &s, const uint64_t *arr, uint32_t cnt0, u128 mass0,
                                              uint64_t top_k, uint32_t ex, int lane, int wave)
{
    if (wave == 0) {
        const uint64_t w0 = arr[127 - 2 * lane], w1 = arr[126 - 2 * lane];
        const uint32_t c0 = pack_count(w0), c1 = pack_count(w1);
        const u128 m0 = pack_mass(w0, ex), m1 = pack_mass(w1, ex);
        const uint32_t cs = c0 + c1;
        const u128 ms = m0 + m1;
        const u128 mi = wave_inclusive_scan(ms);
        const uint32_t ci = wave_inclusive_scan(cs);
        const u128 P = s.P;
        const uint64_t r0 = (uint64_t)cnt0 + ci - cs;      // before my first bin
        const u128 q0 = mass0 + mi - ms;
        const uint64_t r1 = r0 + c0, r2 = r1 + c1;         // before my second bin, after it
        const u128 q1 = q0 + m0, q2 = q1 + m1;
        const bool s0 = r0 >= top_k || q0 >= P, s1 = r1 >= top_k || q1 >= P, s2 = r2 >= top_k || q2 >= P;
        if (!s0 && s1) {
            s.found.bin = 127u - 2u * (uint32_t)lane;
            s.found.cnt_above = (uint32_t)r0; s.found.cnt_bin = c0; s.found.mass_above = q0;
        } else if (!s1 && s2) {
            s.found.bin = 126u - 2u * (uint32_t)lane;
            s.found.cnt_above = (uint32_t)r1; s.found.cnt_bin = c1; s.found.mass_above = q1;
        }
    }
    __syncthreads();
    return s.found;
}

// Mass of this workgroup's own tokens in the bins above index `bin` of a
// 128-bin level (larger e), from s.hm, summed over the workgroup.  All tokens
// of the level share the exponent ex.
__device__ __forceinline__ u128 local_mass_above(Lds &s, uint32_t bin, uint32_t ex, int lane, int wave)
{
    u128 a = 0;
    for (uint32_t b = bin + 1 + threadIdx.x; b <= kTopN; b += kThreads) {
        const uint64_t w = s.hm[b];
        if (w) a += pack_mass(w, ex);
    }
    return block_sum_u128(s, a, lane, wave);
}

// A 124-bit mass in two self-validating words (62 bits each | kValid).
__device__ __forceinline__ void put_mass(uint64_t *slot, u128 v)
{
    a_store(&slot[0], (uint64_t)(((uint64_t)v & ((1ull << 62) - 1)) | kValid));
    a_store(&slot[1], (uint64_t)((uint64_t)(v >> 62) | kValid));
}
__device__ __forceinline__ u128 get_mass(uint64_t w0, uint64_t w1)
{
    return ((u128)(w1 & ~kValid) << 62) | (w0 & ~kValid);
}

// Last act of a workgroup of the cluster kernel: the workgroup that leaves last
// resets the launch-wide counters for the next call.
__device__ __forceinline__ void leave_launch(WsHeader *hdr)
{
    if (threadIdx.x == 0) {
        wait_vmem();
        const uint32_t fin = __hip_atomic_fetch_add(&hdr->finished, 1u, __ATOMIC_RELAXED, RS_AGENT);
        if (fin == gridDim.x - 1) { a_store(&hdr->finished, 0u); a_store(&hdr->ticket, 0u); a_store(&hdr->n_need, 0u); }
    }
}

// Tie weight, kept total S and inverse-CDF target r from the threshold and
// the masses around it (reference: sampling.cu:365-371 and :374-381).  One
// thread; also fills the diagnostics record when there is one.
struct Target { uint64_t w_tie; u128 r; };
__device__ inline Target tie_and_target(const Params &p, uint32_t row, uint64_t rand64, float xmax, u128 D, u128 P,
                                        uint32_t thr, uint32_t n_gt, uint32_t n_eq, u128 Gm, uint32_t levels, bool write_diag)
{
    const uint64_t w_thr = w_of_bits(thr);
    u128 a = (P > Gm) ? (P - Gm) : (u128)0;
    u128 bk = ((uint32_t)p.top_k > n_gt) ? (u128)w_thr * ((uint32_t)p.top_k - n_gt) : (u128)0;
    if (n_eq > 1) { a = div_u32(a, n_eq); bk = div_u32(bk, n_eq); }
    u128 wt = w_thr;
    if (a < wt) wt = a;
    if (bk < wt) wt = bk;
    if (wt == 0 && Gm == 0) wt = 1;
    Target t;
    t.w_tie = (uint64_t)wt;
    const u128 S = Gm + (u128)n_eq * t.w_tie;
    t.r = p.inj_u ? ceil_mul(p.inj_u[row], S) : r_from_bits(rand64, S);
    if (p.diag && write_diag) {
        rs_row_diag *d = p.diag + row;
        d->xmax = xmax; d->emin_bits = 0;
        d->D[0] = (uint64_t)D; d->D[1] = (uint64_t)(D >> 64); d->P[0] = (uint64_t)P; d->P[1] = (uint64_t)(P >> 64);
        d->left_bits = thr; d->thr_bits = thr; d->rounds = levels; d->n_gt = n_gt; d->n_eq = n_eq;
        d->G[0] = (uint64_t)Gm; d->G[1] = (uint64_t)(Gm >> 64); d->w_tie = t.w_tie;
        d->S[0] = (uint64_t)S; d->S[1] = (uint64_t)(S >> 64); d->r[0] = (uint64_t)t.r; d->r[1] = (uint64_t)(t.r >> 64);
    }
    return t;
}

// Waves per SIMD the register allocation must leave room for: the resident
// tokens take 4R registers (8R with penalties), the rest is working set.
template <int R, bool PEN> constexpr int min_waves()
{
    constexpr int data = (PEN ? 8 : 4) * R;
    return data <= 32 ? 4 : data <= 64 ? 3 : 2;
}

// One slice of one row, start to finish.  Returns false when a bounded wait
// gave up (the error word is set; the workgroup must leave at once).
template <int R, bool PEN>
__device__ __forceinline__ bool sample_slice(const Params &p, Lds &s, const uint32_t row, const uint32_t part)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = p.G;
    if (tid == 64 && !p.inj_u) {
        // this call's 64 random bits, drawn while the logits are in flight (the state is
        // advanced once, at the end, by the row's first workgroup)
        const uint32_t *st = p.rng + (size_t)row * 16;
        uint32_t o[4];
        philox4x32_10(st[2], st[3], st[4], st[5], st[0], st[1], o);
        s.bc64[5] = ((uint64_t)o[0] << 32) | o[1];
    }
    RowCtl *rc = p.ctl_end - 1 - row;

    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + (uint32_t)tid;
    // float4 slots of this thread: base4 + j*256, valid while < V4 (a prefix of j)
    const int nv = base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - base4 + kThreads - 1) / kThreads);

    const char *lrow = logits_row(p, row);
    float4 *pn4 = PEN ? reinterpret_cast<float4 *>(p.penalties + (int64_t)row * p.V) : nullptr;

    uint32_t eb[R * 4];                                 // l, then x, then bits(e)
    float4 pen[PEN ? R : 1];

    // ---- 1. load once, scale, local max ---------------------------------
    uint32_t kmax_row;
    {
        if (p.dtype == RS_DTYPE_F32) {
            const float4 *lg = reinterpret_cast<const float4 *>(lrow);
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const uint32_t i4 = min(base4 + (uint32_t)(j * kThreads), V4 - 1);
                const float4 l = lg[i4];
                eb[j * 4 + 0] = __float_as_uint(l.x); eb[j * 4 + 1] = __float_as_uint(l.y);
                eb[j * 4 + 2] = __float_as_uint(l.z); eb[j * 4 + 3] = __float_as_uint(l.w);
                if (PEN) pen[j] = pn4[i4];
            }
        } else {
            const uint2 *lh = reinterpret_cast<const uint2 *>(lrow);
            uint2 h[R];
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const uint32_t i4 = min(base4 + (uint32_t)(j * kThreads), V4 - 1);
                h[j] = lh[i4];
                if (PEN) pen[j] = pn4[i4];
            }
#pragma unroll
            for (int j = 0; j < R; ++j) widen4(h[j], p.dtype, &eb[j * 4]);
        }
        // Fast path: x = (l - pen) * c with no clean-up.  A NaN or Inf anywhere
        // in l, pen or the product shows as a NaN or Inf x, and only then do the
        // sf() calls of the definition change anything.
        // Found at half an instruction per token: a NaN or an infinity among the factors makes
        // the running sum of products NaN or infinite for good (so does an overflow of finite
        // products, which only costs the slow path).
        constexpr int kSpecial = 0x207;                 // sNaN | qNaN | -Inf | +Inf
        float probe = 0.0f;
        float lmax = -3.402823466e+38f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            float x[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float l = __uint_as_float(eb[j * 4 + k]);
                const float pk = PEN ? (k == 0 ? pen[j].x : k == 1 ? pen[j].y : k == 2 ? pen[j].z : pen[j].w) : 0.0f;
                x[k] = PEN ? (l - pk) * p.c : l * p.c;
                eb[j * 4 + k] = __float_as_uint(x[k]);
            }
            probe = __builtin_fmaf(x[0], x[1], probe);
            probe = __builtin_fmaf(x[2], x[3], probe);
            // slots past the end of the row hold its last group again (same slice): harmless here
            lmax = fmaxf(fmaxf(lmax, x[0]), fmaxf(x[1], fmaxf(x[2], x[3])));
        }
        const bool special = __builtin_amdgcn_classf(probe, kSpecial);
        if (special) {
            // Apply the definition with its clean-ups.  Without penalties that is sf of the product
            // already in the registers (sampling.cu:553: masked vocabularies, logits at -inf, end
            // here on every call, so nothing is fetched again); with penalties the logit itself is
            // cleaned first (sampling.cu:220) and has to be read once more.
            lmax = -3.402823466e+38f;
#pragma unroll
            for (int j = 0; j < R; ++j) {
                float x0, x1, x2, x3;
                if (PEN) {
                    const uint32_t i4 = min(base4 + (uint32_t)(j * kThreads), V4 - 1);
                    const float4 l = load_logits4(lrow, i4, p.dtype);
                    x0 = sf((sf(l.x) - pen[j].x) * p.c); x1 = sf((sf(l.y) - pen[j].y) * p.c);
                    x2 = sf((sf(l.z) - pen[j].z) * p.c); x3 = sf((sf(l.w) - pen[j].w) * p.c);
                } else {
                    x0 = sf(__uint_as_float(eb[j * 4])); x1 = sf(__uint_as_float(eb[j * 4 + 1]));
                    x2 = sf(__uint_as_float(eb[j * 4 + 2])); x3 = sf(__uint_as_float(eb[j * 4 + 3]));
                }
                if (j < nv) lmax = fmaxf(lmax, fmaxf(fmaxf(x0, x1), fmaxf(x2, x3)));
                eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
                eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
            }
        }
        kmax_row = block_max_u32(s, fkey(lmax), lane, wave);            // of this slice, for now
        for (int b = tid; b < kNB * kRepC; b += kThreads) s.hr[b] = 0;
        // every workgroup posts its key (never 0 for a finite x) in its own slot
        if (G > 1 && tid == 0) a_store(&rc->mx[part], kmax_row);
        __syncthreads();
    }
    // ---- 2. e in the slice's own frame; level-1 histogram --------------------
    // The significand of e does not depend on the frame, so the row's maximum is not needed
    // yet: bins are kept by absolute octave (mod 128, 4 bins each), where the slices' bins
    // add up as long as their maxima lie within 86 octaves of each other.  The maxima come
    // back with the histogram, in the same polling rounds.
    const float Mloc = __builtin_floorf(fkey_inv(kmax_row));
    const uint32_t pos0 = G > 1 ? (uint32_t)(int)(Mloc - 128.0f * __builtin_floorf(Mloc * 0.0078125f)) * 4u - 508u : 0u;
#pragma unroll
    for (int j = 0; j < R; ++j) {
#pragma unroll
        for (int k = 0; k < 4; ++k) eb[j * 4 + k] = e_bits_of(__uint_as_float(eb[j * 4 + k]), Mloc);
        if (j < nv) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t b = eb[j * 4 + k];
                atomicAdd(reinterpret_cast<unsigned long long *>(&s.hr[(((b >> 21) + pos0) & 511u) * kRepC + (lane & (kRepC - 1))]),
                          (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < kNB / kThreads; ++h) {
        uint64_t w = 0;
#pragma unroll
        for (int c = 0; c < kRepC; ++c) w += s.hr[(tid + h * kThreads) * kRepC + c];
        s.hm[tid + h * kThreads] = w;
    }
    // Cluster histograms this row has used and not yet cleared (bit i: rc->h[i]).  A workgroup may
    // clear its share of one only when every workgroup of the cluster has finished reading it,
    // and only an exchange in which every workgroup publishes something proves that: a deeper
    // histogram level does not, since a slice without tokens in the boundary bin adds nothing to it
    // and the others get past that level without it.
    uint32_t h_used = G > 1 ? 1u : 0u;
    bool mx_posted = G > 1;                              // my slot is still to be cleared
    auto clear_used = [&]() {
        for (uint32_t i = 0; i <= (uint32_t)kLevels; ++i)
            if (h_used >> i & 1u) zero_slice(rc->h[i], (i == 0u || i == (uint32_t)kLevels) ? (uint32_t)kNB : 128u, part, G);
        h_used = 0u;
        if (mx_posted && tid == 0) a_store(&rc->mx[part], 0u);
        mx_posted = false;
    };
    if (G == 1) {
        if (!hist_combine(s, p.hdr, G, rc->h[0], kNB, (uint32_t)p.V, lane, wave)) return false;
    } else {
        const int st = combine_level1(s, p.hdr, G, rc->h[0], rc->mx, (uint32_t)p.V, kmax_row, lane, wave);
        if (st < 0) return false;
        // the row's frame, and this slice's distance from it
        const float dd = __builtin_floorf(fkey_inv(kmax_row)) - Mloc;
        const uint32_t delta = dd >= 64.0f ? 64u : (uint32_t)dd;
        if (delta) {
#pragma unroll
            for (int j = 0; j < R; ++j)
#pragma unroll
                for (int k = 0; k < 4; ++k) eb[j * 4 + k] = rebase_bits(eb[j * 4 + k], delta);
        }
        if (st == 1) {
            // maxima too far apart for the shared octave positions: level 1 again, in the row's
            // frame, through the spare histogram
            __syncthreads();
            lds_hist_zero(s, kNB);
            __syncthreads();
#pragma unroll
            for (int j = 0; j < R; ++j)
                if (j < nv) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t b = opaque(eb[j * 4 + k]);
                        lds_hist_add(s, b >> 21, b);
                    }
                }
            if (!hist_combine(s, p.hdr, G, rc->h[kLevels], kNB, (uint32_t)p.V, lane, wave)) return false;
            // every workgroup has read the first histogram and the slots: it published this one
            // (every slice holds tokens) after that
            clear_used();
            h_used = 1u << kLevels;
        }
    }
    if (p.e_bits) {
        uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) {
                // dead tokens are reported as e = 0
                auto live = [](uint32_t b) { return b < kEMinBits ? 0u : b; };
                dst[base4 + j * kThreads] = make_uint4(live(eb[j * 4]), live(eb[j * 4 + 1]), live(eb[j * 4 + 2]), live(eb[j * 4 + 3]));
            }
    }
    const float xmax = fkey_inv(kmax_row);
    const uint64_t top_k = (uint64_t)p.top_k;

    // ---- 3. radix selection of the threshold -------------------------------
    Found f = hist_find_level1<true>(s, top_k, p.top_p, lane, wave);
    const u128 D = s.D, P = s.P;
    const uint32_t exb = f.bin >> 2;                     // exponent of every token still in play
    // my own tokens: mass in the bins above the boundary, count in the boundary bin
    u128 amass = f.local_above;
    uint32_t mycnt = pack_count(s.hm[f.bin]);
    // bit patterns of the tokens still undistinguished: [lo, lo + span]
    uint32_t lo = f.bin << 21;
    uint32_t span = (1u << 21) - 1u;
    uint32_t levels = 1;                                 // histogram levels summed over the cluster
    // more tokens in the boundary bin than can be gathered, all equal to the row's largest (rows of
    // equal logits): the threshold is that value, no further level is needed
    bool one_tie = false;
    if (f.cnt_bin > (uint32_t)kCap && f.cnt_above == 0u) {
        const uint32_t emax = e_bits_of(xmax, __builtin_floorf(xmax));
        one_tie = bin_is_one_tie(s.g[f.bin], f.bin, emax);
        if (one_tie) { lo = emax; span = 0u; }
    }
    while (!one_tie && f.cnt_bin > (uint32_t)kCap && levels < (uint32_t)kLevels) {
        ++levels;
        const uint32_t dsh = level_shift(levels);
        const uint32_t expect = f.cnt_bin;
        __syncthreads();
        lds_hist_zero(s, 128);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t b = opaque(eb[j * 4 + k]);
                    if (b - lo <= span) lds_hist_add(s, (b >> dsh) & 127u, b);
                }
            }
        if (!hist_combine(s, p.hdr, G, rc->h[levels - 1], 128, expect, lane, wave)) return false;
        if (G > 1) h_used |= 1u << (levels - 1);
        f = hist_find128(s, s.g, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
        amass += local_mass_above(s, f.bin, exb, lane, wave);
        mycnt = pack_count(s.hm[f.bin]);
        lo |= f.bin << dsh;
        span = (1u << dsh) - 1u;
    }

    // If the undistinguished tokens are few, gather them (bits and index) so
    // that every workgroup can finish alone.  Validity is in the data: a
    // gathered entry is never 0, and the words of A[] carry kValid.
    const bool gather = f.cnt_bin <= (uint32_t)kCap;
    const uint32_t ncand = gather ? f.cnt_bin : 0u;
    u128 a_mine = 0;                                     // thread t < G: mass above the bin in workgroup t
    if (gather) {
        __syncthreads();
        if (tid == 0) {
            s.ctr = 0;
            if (G > 1) {
                s.bc32[2] = mycnt ? __hip_atomic_fetch_add(&rc->cursor, mycnt, __ATOMIC_RELAXED, RS_AGENT) : 0u;
                put_mass(&rc->A[2 * part], amass);
            }
        }
        __syncthreads();
        const uint32_t gbase = G > 1 ? s.bc32[2] : 0u;
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t b = opaque(eb[j * 4 + k]);
                    if (b - lo <= span) {
                        const uint32_t o = gbase + atomicAdd(&s.ctr, 1u);
                        const uint32_t idx = (base4 + (uint32_t)j * kThreads) * 4 + (uint32_t)k;
                        const uint64_t cd = ((uint64_t)b << 32) | idx;
                        if (o < (uint32_t)kCap) { if (G > 1) a_store(&rc->cand[o], cd); else s.cand[o] = cd; }
                    }
                }
            }
        if (G > 1) {
            uint64_t w0 = 0, w1 = 0;
            SpinGuard guard;
            guard.start();
            for (;;) {
                uint32_t valid = 0;
                for (uint32_t i = tid; i < ncand; i += kThreads) {
                    const uint64_t w = a_load(&rc->cand[i]);
                    s.cand[i] = w;
                    valid += w != 0;
                }
                if ((uint32_t)tid < G) {
                    w0 = a_load(&rc->A[2 * tid]); w1 = a_load(&rc->A[2 * tid + 1]);
                    valid += (w0 & w1 & kValid) != 0;
                }
                guard.tick(s, p.hdr);
                const uint32_t total = block_sum_u32(s, valid, lane, wave);
                if (total == ncand + G) break;
                if (s.abort) return false;
            }
            if ((uint32_t)tid < G) a_mine = get_mass(w0, w1);
            // every workgroup wrote its mass after it had read the last histogram level
            clear_used();
        } else a_mine = tid == 0 ? amass : (u128)0;
        __syncthreads();

        // resolve the remaining digits on the gathered tokens, in LDS; a single token left in
        // the range is the threshold itself
        for (uint32_t lv = levels + 1; lv <= (uint32_t)kLevels && f.cnt_bin > 1u; ++lv) {
            const uint32_t dsh = level_shift(lv);
            lds_hist_zero(s, 128);
            __syncthreads();
            for (uint32_t i = tid; i < ncand; i += kThreads) {
                const uint32_t b = (uint32_t)(s.cand[i] >> 32);
                if (b - lo <= span) lds_hist_add(s, (b >> dsh) & 127u, b);
            }
            __syncthreads();
            f = hist_find128(s, s.hm, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
            lo |= f.bin << dsh;
            span = (1u << dsh) - 1u;
        }
        if (span != 0u) {
            for (uint32_t i = tid; i < ncand; i += kThreads) {
                const uint32_t b = (uint32_t)(s.cand[i] >> 32);
                if (b - lo <= span) s.bc32[6] = b;
            }
            __syncthreads();
            lo = s.bc32[6];
        }
    }
    // every digit is known: the threshold is the one value left in [lo, lo + span]
    const uint32_t thr = lo;
    const uint32_t n_gt = f.cnt_above, n_eq = f.cnt_bin;
    const u128 Gm = f.mass_above;

    // ---- 5. tie weight, total S, target r (every workgroup, identically) ----
    if (tid == 0) {
        const Target t = tie_and_target(p, row, s.bc64[5], xmax, D, P, thr, n_gt, n_eq, Gm, levels, part == 0);
        s.bc64[1] = t.w_tie; s.bc128[0] = t.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    const u128 r = s.bc128[0];

    // ---- 6. inverse CDF: which workgroup, which float4 slot, which thread ---
    auto weight = [&](uint32_t b) -> uint64_t {
        b = opaque(b);
        return (b > thr) ? w_of_bits(b) : (b == thr ? w_tie : 0);
    };
    auto slot_weight = [&](int j) -> u128 {             // weight of float4 slot j of this thread
        return (u128)weight(eb[j * 4]) + weight(eb[j * 4 + 1]) + weight(eb[j * 4 + 2]) + weight(eb[j * 4 + 3]);
    };
    u128 before = 0, wblock = 0;
    if (gather) {
        // kept weight of workgroup g = mass above the bin in g + weights of its gathered tokens
        const uint32_t shift = 2 + 8 + (uint32_t)__builtin_ctz((unsigned)R);   // token index -> workgroup
        u128 cb = 0, cm = 0;
        for (uint32_t i = tid; i < ncand; i += kThreads) {
            const uint64_t cd = s.cand[i];
            const uint32_t g = ((uint32_t)cd) >> shift;
            const uint64_t w = weight((uint32_t)(cd >> 32));
            if (g < part) cb += w;
            if (g == part) cm += w;
        }
        if ((uint32_t)tid < part) cb += a_mine;
        if ((uint32_t)tid == part) cm += a_mine;
        block_sum2_u128(s, cb, cm, lane, wave);
        before = cb; wblock = cm;
    } else {
        u128 wloc = 0;
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) wloc += slot_weight(j);
        wblock = block_sum_u128(s, wloc, lane, wave);
        if (G > 1) {
            // exchange the kept weights through A[]
            if (tid == 0) put_mass(&rc->A[2 * part], wblock);
            uint64_t w0 = 0, w1 = 0;
            SpinGuard guard;
            guard.start();
            for (;;) {
                uint32_t valid = 0;
                if ((uint32_t)tid < G) {
                    w0 = a_load(&rc->A[2 * tid]); w1 = a_load(&rc->A[2 * tid + 1]);
                    valid = (w0 & w1 & kValid) != 0;
                }
                guard.tick(s, p.hdr);
                const uint32_t total = block_sum_u32(s, valid, lane, wave);
                if (total == G) break;
                if (s.abort) return false;
            }
            clear_used();
            before = block_sum_u128(s, (uint32_t)tid < part ? get_mass(w0, w1) : (u128)0, lane, wave);
        }
    }
    const bool owner = before < r && r <= before + wblock;   // block-uniform

    if (owner) {
        u128 rl = r - before;                            // 1 <= rl <= wblock
        // totals per float4 slot j over the workgroup
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const u128 t = wave_sum(j < nv ? slot_weight(j) : (u128)0);
            if (lane == 0) s.wj[wave][j] = t;
        }
        __syncthreads();
        if (tid < R) { u128 t = 0; for (int w = 0; w < kWaves; ++w) t += s.wj[w][tid]; s.tj[tid] = t; }
        __syncthreads();
        int jstar = 0;
        for (int j = 0; j < R - 1; ++j) { const u128 t = s.tj[j]; if (rl > t) { rl -= t; jstar = j + 1; } else break; }
        // rl <= wblock = sum of tj, so rl now lies inside slot jstar
        uint32_t e4[4] = {0, 0, 0, 0};
        bool have = false;
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j == jstar) { have = j < nv; e4[0] = eb[j * 4]; e4[1] = eb[j * 4 + 1]; e4[2] = eb[j * 4 + 2]; e4[3] = eb[j * 4 + 3]; }
        const u128 w0 = have ? weight(e4[0]) : 0, w1 = have ? weight(e4[1]) : 0;
        const u128 w2 = have ? weight(e4[2]) : 0, w3 = have ? weight(e4[3]) : 0;
        const u128 mine = w0 + w1 + w2 + w3;
        // inclusive scan over the 256 threads of slot jstar
        u128 inc = wave_inclusive_scan(mine);
        __syncthreads();
        if (lane == kWave - 1) s.q128[wave] = inc;
        __syncthreads();
        u128 woff = 0;
        for (int w = 0; w < wave; ++w) woff += s.q128[w];
        inc += woff;
        const u128 exc_ = inc - mine;
        if (exc_ < rl && rl <= inc) {                     // exactly one thread
            const u128 rr = rl - exc_;                    // 1 <= rr <= mine
            const int kk = (rr <= w0) ? 0 : (rr <= w0 + w1) ? 1 : (rr <= w0 + w1 + w2) ? 2 : 3;
            const int32_t idx = (int32_t)((base4 + (uint32_t)jstar * kThreads) * 4 + (uint32_t)kk);
            p.out[row] = idx;
            if (p.diag) p.diag[row].index = idx;
            if (PEN && G > 1) a_store(&rc->index_p1, (uint32_t)idx + 1u);
            if (PEN) s.bc32[7] = (uint32_t)idx;
        }
    }

    // ---- 7. penalties: decay and one-hot add, from registers ---------------
    if (PEN) {
        __syncthreads();
        if (G > 1) {
            if (tid == 0) {
                const uint64_t t0 = wall_clock64();
                uint32_t spins = 0, v;
                while ((v = a_load(&rc->index_p1)) == 0u) {
                    if ((++spins & 1023u) == 0 && (uint64_t)wall_clock64() - t0 > spin_limit(p.hdr)) {
                        give_up(s, p.hdr);
                        break;
                    }
                }
                s.bc32[7] = v - 1u;
            }
            __syncthreads();
            if (s.abort) return false;
        }
        const uint32_t idx = s.bc32[7];
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j < nv) {
                const uint32_t i4 = base4 + (uint32_t)j * kThreads;
                float4 v = pen[j];
                const uint32_t e0 = i4 * 4;
                v.x = __builtin_fmaf(v.x, p.decay, (e0 + 0 != idx) ? 0.0f : (v.x == 0.0f ? p.presence : p.repetition));
                v.y = __builtin_fmaf(v.y, p.decay, (e0 + 1 != idx) ? 0.0f : (v.y == 0.0f ? p.presence : p.repetition));
                v.z = __builtin_fmaf(v.z, p.decay, (e0 + 2 != idx) ? 0.0f : (v.z == 0.0f ? p.presence : p.repetition));
                v.w = __builtin_fmaf(v.w, p.decay, (e0 + 3 != idx) ? 0.0f : (v.w == 0.0f ? p.presence : p.repetition));
                pn4[i4] = v;
            }
        }
    }

    // ---- leave: advance the RNG, clean the row record, reset the launch ----
    __syncthreads();
    if (G > 1) {
        if (tid == 0) s.bc32[0] = __hip_atomic_fetch_add(&rc->done, 1u, __ATOMIC_RELAXED, RS_AGENT);
        __syncthreads();
        if (s.bc32[0] == G - 1) {
            // last workgroup out of this row: nobody reads the record any more
            for (uint32_t i = tid; i < ncand; i += kThreads) a_store(&rc->cand[i], (uint64_t)0);
            if ((uint32_t)tid < G) { a_store(&rc->A[2 * tid], (uint64_t)0); a_store(&rc->A[2 * tid + 1], (uint64_t)0); }
            if (tid == 0) { a_store(&rc->done, 0u); a_store(&rc->cursor, 0u); a_store(&rc->index_p1, 0u); }
        }
    }
    if (tid == 0) {
        if (part == 0 && !p.inj_u) {
            uint32_t *st = p.rng + (size_t)row * 16;
            const uint32_t lo32 = st[2] + 1;
            st[2] = lo32;
            if (lo32 == 0) st[3] += 1;
        }
    }
    return true;
}

// Workgroups take their (row, slice) from a ticket counter, so that logical
// ids follow the order in which workgroups actually start: a workgroup only
// ever waits for lower tickets, whose holders are running or done.
template <int R, bool PEN>
__global__ void __launch_bounds__(kThreads, (min_waves<R, PEN>())) sample_kernel(const Params p)
{
    __shared__ Lds s;
    if (p.G == 1) {
        // one workgroup per row: nobody waits for anybody, the hardware's ids will do
        if (threadIdx.x == 0) { s.abort = 0; s.host_words = p.host_words; }
        __syncthreads();
        sample_slice<R, PEN>(p, s, blockIdx.x, 0u);
        return;
    }
    if (threadIdx.x == 0) {
        s.abort = 0; s.host_words = p.host_words;
        const uint32_t t = __hip_atomic_fetch_add(&p.hdr->ticket, 1u, __ATOMIC_RELAXED, RS_AGENT);
        // every workgroup of the launch takes exactly one ticket: after the last one the counter
        // is not touched again, and is put back for the next call
        if (t == gridDim.x - 1) a_store(&p.hdr->ticket, 0u);
        s.bc32[0] = t;
    }
    __syncthreads();
    const uint32_t ticket = s.bc32[0];
    const uint32_t row = ticket / p.G;
    sample_slice<R, PEN>(p, s, row, ticket - row * p.G);
}

// The launch that follows the streaming pass knows how many rows were handed on.  Its first
// workgroup tells the host -- a word of pinned memory that rs_sample looks at, without waiting,
// before its next call -- whether that was most of them: such calls are then better served by
// the cluster kernel alone for a while.  The word belongs to the caller's rs_policy.
__device__ __forceinline__ void report_streaming(const Params &p, uint32_t handed_on)
{
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.host_words)
        __hip_atomic_store(p.host_words + p.report, handed_on * 2u > (uint32_t)p.B ? 1 : 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The launch that follows the streaming pass: workgroups work through the
// rows on its list, taking tickets until the list is exhausted.
template <int R>
__global__ void __launch_bounds__(kThreads, (min_waves<R, false>())) sample_list_kernel(const Params p)
{
    __shared__ Lds s;
    const uint32_t G = p.G;
    const uint32_t n = a_load(&p.hdr->n_need);
    report_streaming(p, n);
    if (n == 0u) return;                                         // nothing left over: no ticket was taken
    for (;;) {
        __syncthreads();
        if (threadIdx.x == 0) {
            s.abort = 0; s.host_words = p.host_words;
            s.bc32[0] = __hip_atomic_fetch_add(&p.hdr->ticket, 1u, __ATOMIC_RELAXED, RS_AGENT);
        }
        __syncthreads();
        const uint32_t ticket = s.bc32[0];
        const uint32_t slot = ticket / G;
        if (slot >= a_load(&p.hdr->n_need)) break;
        if (!sample_slice<R, false>(p, s, p.need[slot], ticket - slot * G)) return;
    }
    leave_launch(p.hdr);
}

// The same for a launch of one workgroup per slice of every row of the batch:
// each takes one ticket, those beyond the list leave at once.  Used behind an
// attempt, after which the list may hold every row.
template <int R>
__global__ void __launch_bounds__(kThreads, (min_waves<R, false>())) sample_list_once_kernel(const Params p)
{
    __shared__ Lds s;
    const uint32_t n = a_load(&p.hdr->n_need);
    report_streaming(p, n);
    if (n == 0u) return;                                         // nothing left over: no ticket was taken
    if (threadIdx.x == 0) {
        s.abort = 0; s.host_words = p.host_words;
        const uint32_t t = __hip_atomic_fetch_add(&p.hdr->ticket, 1u, __ATOMIC_RELAXED, RS_AGENT);
        if (t == gridDim.x - 1) a_store(&p.hdr->ticket, 0u);     // the last ticket of the launch
        s.bc32[0] = t;
    }
    __syncthreads();
    const uint32_t ticket = s.bc32[0];
    const uint32_t slot = ticket / p.G;
    if (slot >= n) return;
    sample_slice<R, false>(p, s, p.need[slot], ticket - slot * p.G);
}

// ---------------------------------------------------------- streaming path --
// When the kept set is small next to the row the cluster kernel's exchanges
// cost more than the data movement.  The streaming path has no waits at all:
//
//   stream_kernel   one workgroup per slice.  It reads the slice once, takes
//                   its OWN maximum as the frame (the significand of e does
//                   not depend on the frame, so a slice's histogram is the
//                   row's up to a shift of whole octaves), adds its level-1
//                   histogram to the row's and stashes its largest tokens --
//                   several times its share of the row's top_k -- ordered by
//                   bin, with the exact value down to which the stash is
//                   complete.
//   finish_kernel   one workgroup per row.  It brings the row's histogram into
//                   the row's frame, finds the boundary bin, pulls the stashed
//                   tokens at or above it (or, for flat rows, the stashes
//                   whole), resolves the threshold on them and picks.  A row
//                   that cannot be finished from the stashes (a huge tie, a
//                   nucleus of thousands of tokens) is put on a list, and the
//                   cluster kernel then runs for the listed rows.
constexpr int      kSB       = 164;           // level-1 bins in use: indices 348..511
constexpr int      kStashCap = 1280;          // stash entries per slice (at least kStreamK)
constexpr int      kStreamK  = 1024;          // largest top_k the streaming path takes
constexpr int      kFinCap   = 8192;          // tokens the finishing workgroup can hold at most (64 KB of LDS)

struct PartHdr {
    uint32_t mkey;        // fkey(max x of the slice)
    uint32_t cov;         // the stash holds every token of the slice with bin - 348 >= cov
    uint32_t n;           // entries in the stash
    uint32_t cut;         // the stash holds every token of the slice with bits(e) >= cut (slice frame); cut lies in
                          // bin cov or, when only part of a bin fitted, in bin cov - 1
};

struct StreamView {
    PartHdr  *hdr;        // [B][G]
    uint64_t *stash;      // [B][G][kStashCap]   bits(e, slice frame) << 32 | index, by descending bin
    uint32_t *cum;        // [B][G][kSB]   tokens of the slice in this bin and the bins above it
    uint64_t *shist;      // [B][G][kSB]   the slice's own bins (slice frame), as it added them to the row's
    uint32_t *need;       // [B]  rows left to the cluster kernel
    uint32_t  G;          // slices per row
    uint32_t  list_cap;   // entries of the finishing workgroup's token list (a power of two up to kFinCap)
};

// Lanes of a wave that add to one LDS address are served one after the other, and rows often put
// most of their tokens into a few bins.  So each bin is kept in kRep copies (lane l adds to copy
// l % kRep), and e is not clamped before it is counted: the histogram spans all 512 values of
// bits >> 21, the dead tokens (below 2^-40, often most of a row) spread over the bins below
// kBin0 by their own exponents, where nobody looks at them again.  The histogram is done with
// before the candidates are staged, and shares their memory.
// Eight copies for long slices; two for the short slices of small calls, where clearing and
// folding the copies would cost more than the few tokens of a thread.
template <int R> constexpr int stream_copies() { return R >= 8 ? 8 : 2; }
template <int kRep>
struct LdsA {
    union {
        uint64_t hm[kNB * kRep];     // the slice's bins by bits >> 21
        struct {
            uint4    grp[kStashCap];     // float4 groups that hold a candidate: bits of their 4 tokens
            uint32_t gidx[kStashCap];    // and the index of their first token
        };
    };
    uint32_t off[kSB];
    uint32_t sub[128];           // level-2 counts inside a boundary bin too large for the stash
    uint32_t u32[16];
    uint32_t cov, n, cut, over;
};

template <int R, int NT, int DT>     // NT threads, each with R groups of four tokens of the slice; DT the logits' type
__global__ void __launch_bounds__(NT, (R <= 8 ? 5 : 3)) stream_kernel(const Params p, const StreamView v)
{
    constexpr int kRep = stream_copies<R>();
    __shared__ LdsA<kRep> s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t base4 = part * (uint32_t)(NT * R) + (uint32_t)tid;
    const int nv = base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - base4 + NT - 1) / NT);
    const char *lrow = logits_row(p, row);

    uint32_t eb[R * 4];                                 // l, then x, then bits(e)
    // x = l * c is the definition unless a NaN or Inf shows up (see sample_kernel).  Slots past the
    // end of the row read its last group again: harmless for the maximum and the probe, and they
    // are set aside before the histogram.
    constexpr int kSpecial = 0x207;
    float probe = 0.0f;
    float lmax = -3.402823466e+38f;
    if constexpr (DT == RS_DTYPE_F32) {
        const float4 *lg = reinterpret_cast<const float4 *>(lrow);
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const float4 l = lg[min(base4 + (uint32_t)(j * NT), V4 - 1)];
            eb[j * 4 + 0] = __float_as_uint(l.x); eb[j * 4 + 1] = __float_as_uint(l.y);
            eb[j * 4 + 2] = __float_as_uint(l.z); eb[j * 4 + 3] = __float_as_uint(l.w);
        }
    } else {
        const uint2 *lh = reinterpret_cast<const uint2 *>(lrow);
        uint2 h[R];
#pragma unroll
        for (int j = 0; j < R; ++j) h[j] = lh[min(base4 + (uint32_t)(j * NT), V4 - 1)];
#pragma unroll
        for (int j = 0; j < R; ++j) widen4(h[j], DT, &eb[j * 4]);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const float x0 = __uint_as_float(eb[j * 4]) * p.c, x1 = __uint_as_float(eb[j * 4 + 1]) * p.c;
        const float x2 = __uint_as_float(eb[j * 4 + 2]) * p.c, x3 = __uint_as_float(eb[j * 4 + 3]) * p.c;
        probe = __builtin_fmaf(x0, x1, probe);
        probe = __builtin_fmaf(x2, x3, probe);
        lmax = fmaxf(fmaxf(lmax, x0), fmaxf(x1, fmaxf(x2, x3)));
        eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
        eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
    }
    if (__builtin_amdgcn_classf(probe, kSpecial)) {
        // the clean-up of sampling.cu:553 on the products already in the registers (masked
        // vocabularies, logits at -inf, come through here on every call)
        lmax = -3.402823466e+38f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const float x0 = sf(__uint_as_float(eb[j * 4])), x1 = sf(__uint_as_float(eb[j * 4 + 1]));
            const float x2 = sf(__uint_as_float(eb[j * 4 + 2])), x3 = sf(__uint_as_float(eb[j * 4 + 3]));
            if (j < nv) lmax = fmaxf(lmax, fmaxf(fmaxf(x0, x1), fmaxf(x2, x3)));
            eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
            eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
        }
    }
    {
        uint4 *z = reinterpret_cast<uint4 *>(s.hm);                              // two bins per store
#pragma unroll
        for (int i = 0; i < kNB * kRep / 2 / NT; ++i) z[tid + i * NT] = make_uint4(0u, 0u, 0u, 0u);
        static_assert(kNB * kRep % (2 * NT) == 0, "whole stores");
    }
    if (blockIdx.x == 0 && tid == 0) a_store(&p.hdr->n_need, 0u);   // the list of the previous call is history
    uint32_t k = wave_max_u32(fkey(lmax));
    if (lane == 0) s.u32[wave] = k;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < (NT / kWave); ++w) k = max(k, s.u32[w]);
    const float M = __builtin_floorf(fkey_inv(k));

    // e in the slice's frame, not yet clamped at 2^-40, and its histogram; slots past the end of
    // the row become 0
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (j < nv) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t b = e_bits_raw(__uint_as_float(eb[j * 4 + q]), M);
                eb[j * 4 + q] = b;
                atomicAdd(reinterpret_cast<unsigned long long *>(&s.hm[(b >> 21) * kRep + (lane & (kRep - 1))]),
                          (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
            }
        } else {
            eb[j * 4] = 0; eb[j * 4 + 1] = 0; eb[j * 4 + 2] = 0; eb[j * 4 + 3] = 0;
        }
    }
    if (p.e_bits) {
        // diagnostics: e of every token, still in the slice's frame; the finishing workgroup re-bases it
        uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) dst[base4 + j * NT] = make_uint4(eb[j * 4], eb[j * 4 + 1], eb[j * 4 + 2], eb[j * 4 + 3]);
    }
    __syncthreads();
    // Add the slice's live bins to the row's, which are kept by absolute octave (mod 128, 4 bins each):
    // bin t of this frame is octave M - 40 + t/4.  Slices of one row may use different frames; as
    // long as their maxima lie within 87 octaves of each other no two octaves in use coincide.
    auto bin_total = [&](int b) {
        const uint4 *two = reinterpret_cast<const uint4 *>(&s.hm[((int)kBin0 + b) * kRep]);     // two copies per load
        uint64_t w = 0;
#pragma unroll
        for (int c = 0; c < kRep / 2; ++c) {
            const uint4 q = two[c];
            w += (((uint64_t)q.y << 32) | q.x) + (((uint64_t)q.w << 32) | q.z);
        }
        return w;
    };
    if (tid < kSB) {
        const uint64_t w = bin_total(tid);
        const float mm = M - 128.0f * __builtin_floorf(M * 0.0078125f);          // M mod 128, exact
        v.shist[((size_t)row * G + part) * kSB + tid] = w;                        // kept for rows whose slices lie far apart
        if (w) a_add(&(p.ctl_end - 1 - row)->rowhist[((uint32_t)(int)mm * 4u + (uint32_t)tid - 160u) & 511u], w);
    }

    // What to stash: the bins from the top down to the first one at which the count reaches
    // stash_k (that bin too if it fits).  With stash_k = top_k the row's top_k tokens are certainly
    // in the stashes; the host aims lower when a row has many slices, since a slice then holds
    // about top_k / slices of them, and the finishing workgroup checks that each stash reaches
    // down to the row's boundary bin before it relies on it.
    if (wave == 0) {
        const uint32_t Ks = p.stash_k;
        uint32_t c3[3];
        uint32_t cs = 0;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int b = kSB - 1 - 3 * lane - i;
            c3[i] = b >= 0 ? pack_count(bin_total(b)) : 0u;
            cs += c3[i];
        }
        const uint32_t ci = wave_inclusive_scan(cs);
        uint32_t run = ci - cs;
        const uint32_t total = lane63(ci);
        if (lane == 0) s.over = 0xFFFFFFFFu;
        if (lane == 0 && total < Ks) { s.cov = 0u; s.n = total; s.cut = kBin0 << 21; }   // a short slice: all its live tokens
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int b = kSB - 1 - 3 * lane - i;
            const uint32_t nx = run + c3[i];
            if (b >= 0) {
                s.off[b] = run;                                           // tokens in the bins above b
                v.cum[((size_t)row * G + part) * kSB + b] = nx;
            }
            if (run < Ks && nx >= Ks) {
                // the whole bin if that stays close to stash_k, else only part of it (found below)
                if (nx <= min((uint32_t)kStashCap, Ks + max(64u, Ks >> 2))) { s.cov = (uint32_t)b; s.n = nx; s.cut = ((uint32_t)b + kBin0) << 21; }
                else { s.cov = (uint32_t)b + 1u; s.n = run; s.cut = ((uint32_t)b + 1u + kBin0) << 21; s.over = (uint32_t)b; }
            }
            run = nx;
        }
    }
    if (tid < 128) s.sub[tid] = 0;
    __syncthreads();
    if (s.over != 0xFFFFFFFFu) {
        // The bin in which the count reaches stash_k holds far more tokens than asked for (a flat
        // distribution: hundreds or thousands of tokens within a quarter octave).  Look at its next
        // 7 bits and take the sub-bins from the top down to the one at which the count reaches
        // stash_k, as far as they fit.
        const uint32_t ob = s.over + kBin0, above = s.n;
        // a bin that is one tie of the slice's largest token (rows of equal logits) has all its
        // tokens in one sub-bin: known without counting, which would queue them up at one address
        const uint32_t emax = e_bits_raw(fkey_inv(k), M);
        const uint64_t wbin = bin_total((int)s.over);
        if (above == 0u && bin_is_one_tie(wbin, ob, emax)) {
            if (tid == 0) s.sub[(emax >> 14) & 127u] = pack_count(wbin);
        } else {
#pragma unroll
            for (int j = 0; j < R; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t b = eb[j * 4 + q];
                    if ((b >> 21) == ob) atomicAdd(&s.sub[(b >> 14) & 127u], 1u);
                }
        }
        __syncthreads();
        if (wave == 0) {
            const uint32_t Ks = p.stash_k;
            const uint32_t c0 = s.sub[127 - 2 * lane], c1 = s.sub[126 - 2 * lane];
            const uint32_t ci = wave_inclusive_scan(c0 + c1);
            const uint32_t r0 = above + ci - c0 - c1, r1 = r0 + c0, r2 = r1 + c1;
            // first sub-bin at which the count reaches stash_k (there is one: the whole bin reaches it)
            if (r0 < Ks && r1 >= Ks) {
                const bool fits = r1 <= (uint32_t)kStashCap;
                s.n = fits ? r1 : r0;
                s.cut = (ob << 21) + ((127u - 2u * (uint32_t)lane + (fits ? 0u : 1u)) << 14);
            } else if (r1 < Ks && r2 >= Ks) {
                const bool fits = r2 <= (uint32_t)kStashCap;
                s.n = fits ? r2 : r1;
                s.cut = (ob << 21) + ((126u - 2u * (uint32_t)lane + (fits ? 0u : 1u)) << 14);
            }
        }
        __syncthreads();
    }
    const uint32_t cov = s.cov, n = s.n;
    const uint32_t cut = s.cut;
    // From here on the bits in the registers are compared with the cut, which is never below
    // 2^-40: dead tokens are no candidates.

    // Candidates (bits >= cut) are at most n <= kStashCap, so at most that many float4 groups
    // hold one.  Each thread copies its groups with a candidate into LDS at an offset from a scan
    // of the per-thread counts; the tokens of those groups are then gone through densely.
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < R; ++j)
        mine += max(max(eb[j * 4], eb[j * 4 + 1]), max(eb[j * 4 + 2], eb[j * 4 + 3])) >= cut ? 1u : 0u;
    uint32_t o = wave_inclusive_scan(mine);
    if (lane == kWave - 1) s.u32[wave] = o;
    __syncthreads();
    uint32_t ngroups = 0;
#pragma unroll
    for (int w = 0; w < (NT / kWave); ++w) {
        if (w < wave) o += s.u32[w];
        ngroups += s.u32[w];
    }
    o -= mine;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (max(max(eb[j * 4], eb[j * 4 + 1]), max(eb[j * 4 + 2], eb[j * 4 + 3])) >= cut) {
            if (o < (uint32_t)kStashCap) {
                s.grp[o] = make_uint4(eb[j * 4], eb[j * 4 + 1], eb[j * 4 + 2], eb[j * 4 + 3]);
                s.gidx[o] = (base4 + (uint32_t)j * NT) * 4;
            }
            ++o;
        }
    }
    __syncthreads();
    // Write the candidates out grouped by bin, largest e first, so that the finishing
    // workgroup can take a prefix.
    uint64_t *st = v.stash + ((size_t)row * G + part) * kStashCap;
    const uint32_t *gb = reinterpret_cast<const uint32_t *>(s.grp);
#pragma unroll 4
    for (uint32_t i = tid; i < min(ngroups, (uint32_t)kStashCap) * 4u; i += NT) {
        const uint32_t b = gb[i];
        if (b >= cut) {
            const uint32_t slot = atomicAdd(&s.off[(b >> 21) - kBin0], 1u);
            if (slot < (uint32_t)kStashCap) st[slot] = ((uint64_t)b << 32) | (s.gidx[i >> 2] + (i & 3u));
        }
    }
    if (tid == 0) {
        PartHdr ph;
        ph.mkey = k; ph.cov = cov; ph.n = n; ph.cut = cut;
        v.hdr[(size_t)row * G + part] = ph;
    }
}

struct LdsB {
    uint64_t *list;              // gathered tokens, row frame: bits << 32 | index (dynamic LDS, v.list_cap entries)
    uint64_t blo[kMaxParts], bhi[kMaxParts];
    uint64_t small[64];
    uint32_t delta[kMaxParts];   // octaves between the row's frame and slice g's
    uint32_t m4[kMaxParts];      // 4 (M mod 128) of slice g's frame: where its bins sit among the row's positions
    uint32_t take[kMaxParts];    // inclusive prefix of the entries taken from each stash
    uint64_t rand64;
    uint32_t nsmall, bucket, fail;
};

// Inverse CDF by buckets of the token index: sum the kept weights per bucket
// (bucket = (index >> shift) & 255, tokens outside [lo_idx, hi_idx) ignored),
// scan, and return the bucket that holds target r, with r reduced to an offset
// inside it.  Weights are < 2^64 and a sum has < 2^12 terms, so the halves
// summed separately stay below 2^44 + 2^32.
template <typename W>
__device__ __forceinline__ uint32_t bucket_step(Lds &s, LdsB &t, uint32_t nlist, uint32_t shift, uint32_t lo_idx, uint32_t hi_idx,
                                                u128 &r, W weight, int lane, int wave)
{
    const int tid = threadIdx.x;
    t.blo[tid] = 0; t.bhi[tid] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < nlist; i += kThreads) {
        const uint64_t e = t.list[i];
        const uint32_t idx = (uint32_t)e;
        if (idx >= lo_idx && idx < hi_idx) {
            const uint64_t w = weight((uint32_t)(e >> 32));
            if (w) {
                const uint32_t bk = (idx >> shift) & 255u;
                atomicAdd(reinterpret_cast<unsigned long long *>(&t.blo[bk]), (unsigned long long)(w & 0xFFFFFFFFull));
                atomicAdd(reinterpret_cast<unsigned long long *>(&t.bhi[bk]), (unsigned long long)(w >> 32));
            }
        }
    }
    __syncthreads();
    const u128 mine = (u128)t.blo[tid] + ((u128)t.bhi[tid] << 32);
    u128 inc = wave_inclusive_scan(mine);
    if (lane == kWave - 1) s.q128[wave] = inc;
    __syncthreads();
    for (int w = 0; w < wave; ++w) inc += s.q128[w];
    const u128 exc = inc - mine;
    if (exc < r && r <= inc) { t.bucket = (uint32_t)tid; s.bc128[1] = r - exc; }
    __syncthreads();
    r = s.bc128[1];
    return t.bucket;
}

template <int SLICE_LOG2>     // log2 of the tokens per slice of the view
__device__ __forceinline__ void finish_row(const Params &p, const StreamView &v, Lds &s, LdsB &t, const uint32_t row)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const PartHdr *hdrs = v.hdr + (size_t)row * G;
    uint64_t *rowhist = (p.ctl_end - 1 - row)->rowhist;

    if (tid == 0) { s.abort = 0; s.host_words = p.host_words; t.fail = 0; }
    PartHdr ph;
    ph.mkey = 0; ph.cov = 0; ph.n = 0; ph.cut = 0;
    if ((uint32_t)tid < G) ph = hdrs[tid];
    const uint64_t h0 = rowhist[tid], h1 = rowhist[tid + kThreads];
    // the first lane of wave 1 draws the row's random number while wave 0 scans the histogram;
    // the state is advanced only once the row is certain to be finished here
    const bool drawer = tid == kWave && !p.inj_u;
    uint32_t *rng_st = p.rng + (size_t)row * 16;
    uint32_t rs[6] = {0u, 0u, 0u, 0u, 0u, 0u};
    if (drawer) {
#pragma unroll
        for (int i = 0; i < 6; ++i) rs[i] = rng_st[i];
    }
    rowhist[tid] = 0; rowhist[tid + kThreads] = 0;                   // left clean for the next call
    uint32_t kmax, kmin;
    {
        const uint32_t a = wave_max_u32(ph.mkey), b = wave_max_u32((uint32_t)tid < G ? ~ph.mkey : 0u);
        if (lane == 0) { s.u32[wave] = a; s.u32[kWaves + wave] = b; }
        __syncthreads();
        kmax = s.u32[0]; kmin = s.u32[kWaves];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { kmax = max(kmax, s.u32[w]); kmin = max(kmin, s.u32[kWaves + w]); }
        kmin = ~kmin;
    }
    const float xmax = fkey_inv(kmax);
    const float M = __builtin_floorf(xmax);
    // frames further apart than this may have put different octaves into one bin
    const bool mixed = !(M - __builtin_floorf(fkey_inv(kmin)) < 88.0f);
    uint32_t dl = 0;
    if ((uint32_t)tid < G) {
        const float d = M - __builtin_floorf(fkey_inv(ph.mkey));      // >= 0, a whole number or huge
        dl = d >= 64.0f ? 64u : (uint32_t)d;
        t.delta[tid] = dl;
        const float Mg = __builtin_floorf(fkey_inv(ph.mkey));
        t.m4[tid] = (uint32_t)(int)(Mg - 128.0f * __builtin_floorf(Mg * 0.0078125f)) * 4u;
    }
    // the row's level-1 histogram in the row's frame: bin r (octave M - 40 + r/4) sits at absolute
    // position 4 (M mod 128) + r - 160; the other 348 positions hold tokens below 2^-40 of this
    // frame, which are dead there: dropped
    {
        const float mm = M - 128.0f * __builtin_floorf(M * 0.0078125f);
        const uint32_t m4 = (uint32_t)(int)mm * 4u;
        const uint32_t r0 = ((uint32_t)tid + 160u - m4) & 511u, r1 = ((uint32_t)tid + kThreads + 160u - m4) & 511u;
        if (r0 < (uint32_t)kSB) s.g[kBin0 + r0] = h0;
        if (r1 < (uint32_t)kSB) s.g[kBin0 + r1] = h1;
        for (int b = tid; b < (int)kBin0; b += kThreads) s.g[b] = 0;
        __syncthreads();
        if (mixed) {
            // Slices whose maxima lie 88 octaves or more apart may have put different octaves into
            // one position.  Every token of a slice 41 octaves or more below the row's frame is
            // dead there, whatever its bin: what such a slice added is taken out again, bin by bin
            // (its own bins are on record).  The slices that remain lie within 40 octaves of each
            // other.
            for (uint32_t i = (uint32_t)tid; i < G * (uint32_t)kSB; i += kThreads) {
                const uint32_t g = i / (uint32_t)kSB, r = i - g * (uint32_t)kSB;
                if (t.delta[g] >= 41u) {
                    const uint64_t w = v.shist[((size_t)row * G + g) * kSB + r];
                    if (w) {
                        const uint32_t rr = (t.m4[g] + r - m4) & 511u;
                        if (rr < (uint32_t)kSB)
                            atomicAdd(reinterpret_cast<unsigned long long *>(&s.g[kBin0 + rr]), 0ull - (unsigned long long)w);
                    }
                }
            }
        }
    }
    __syncthreads();
    if (p.e_bits) {
        // diagnostics: the slices' e into the row's frame, dead tokens as 0
        uint4 *eb4 = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
        auto fix = [&](uint32_t b, uint32_t d) { b = rebase_bits(min(b, 0x3FFFFFFFu), d); return b < kEMinBits ? 0u : b; };
        for (uint32_t i4 = (uint32_t)tid; i4 < ((uint32_t)p.V >> 2); i4 += kThreads) {
            const uint32_t d = t.delta[i4 >> (SLICE_LOG2 - 2)];
            uint4 q = eb4[i4];
            q.x = fix(q.x, d); q.y = fix(q.y, d); q.z = fix(q.z, d); q.w = fix(q.w, d);
            eb4[i4] = q;
        }
    }
    if (drawer) {
        uint32_t o[4];
        philox4x32_10(rs[2], rs[3], rs[4], rs[5], rs[0], rs[1], o);
        t.rand64 = ((uint64_t)o[0] << 32) | o[1];
    }
    const uint64_t top_k = (uint64_t)p.top_k;
    Found f = hist_find_level1<false>(s, top_k, p.top_p, lane, wave);
    const u128 D = s.D, P = s.P;

    // A row that is one tie of all its tokens (rows of equal logits) needs no stash at all: the
    // threshold is the largest token's value, every token weighs the tie weight, and the token at
    // which the running sum reaches r follows by division.
    if (f.cnt_bin == (uint32_t)p.V && bin_is_one_tie(s.g[f.bin], f.bin, e_bits_of(xmax, M))) {
        if (drawer) {
            rng_st[2] = rs[2] + 1u;
            if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
        }
        if (tid == 0) {
            const uint32_t thr1 = e_bits_of(xmax, M);
            const Target tg = tie_and_target(p, row, p.inj_u ? 0ull : t.rand64, xmax, D, P, thr1, 0u, f.cnt_bin, (u128)0, 0u, true);
            // smallest i with (i + 1) * w_tie >= r; r <= V * w_tie
            uint32_t lo_i = 0, hi_i = (uint32_t)p.V - 1u;
            while (lo_i < hi_i) {
                const uint32_t mid = (lo_i + hi_i) >> 1;
                if ((u128)(mid + 1u) * tg.w_tie >= tg.r) hi_i = mid; else lo_i = mid + 1u;
            }
            p.out[row] = (int32_t)lo_i;
            if (p.diag) p.diag[row].index = (int32_t)lo_i;
        }
        return;
    }

    // Plan A: every stash reaches down to the row's boundary bin.  Then exactly the tokens at or
    // above that bin are taken, a prefix of each stash whose length is one cumulative count.
    uint32_t total = f.cnt_above + f.cnt_bin;
    uint32_t mtake = 0;
    bool bad = total > v.list_cap;
    if ((uint32_t)tid < G) {
        const int lb = (int)(f.bin - kBin0) + 4 * (int)dl;            // boundary bin in the slice's frame
        if (dl >= 64u) mtake = 0;                                      // the whole slice is dead in the row's frame
        else if (lb < kSB) mtake = v.cum[((size_t)row * G + tid) * kSB + lb];
        if (mtake && ((int)ph.cov > lb || mtake > ph.n)) bad = true;
    }
    if (bad) t.fail = 1;
    auto take_prefix = [&](uint32_t mine) {                           // inclusive prefix over the slices, into t.take
        uint32_t inc = wave_inclusive_scan(mine);
        __syncthreads();
        if (lane == kWave - 1) s.u32[wave] = inc;
        __syncthreads();
        for (int w = 0; w < wave; ++w) inc += s.u32[w];
        t.take[tid] = inc;
        __syncthreads();
    };
    take_prefix(mtake);
    bool subset = false;                                               // plan B in force
    uint32_t cutrow = 0;
    if (t.fail || t.take[kThreads - 1] != total) {
        // Plan B (flat distributions: the boundary bin holds thousands of tokens, but top_k is small):
        // take the stashes whole.  Together they hold every token of the row at or above
        // cutrow = the largest of the slices' cuts, so a threshold found among those is the row's.
        uint32_t mycut = 0;
        if ((uint32_t)tid < G) {
            // a cut that lands below 2^-40 in the row's frame: what the stash lacks is dead there
            mycut = max(rebase_bits(ph.cut, dl), kEMinBits);
        }
        cutrow = block_max_u32(s, mycut, lane, wave);
        take_prefix((uint32_t)tid < G ? min(ph.n, (uint32_t)kStashCap) : 0u);
        total = t.take[kThreads - 1];
        if (total > v.list_cap || total == 0u) {
            // not resolvable from the stashes: leave the row to the cluster kernel
            if (tid == 0) {
                const uint32_t slot = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
                v.need[slot] = row;
            }
            return;
        }
        subset = true;
    }

    // gather the tokens, re-based to the row's frame: a thread takes a run of consecutive list
    // entries, so that it looks up its first slice once and walks on from there
    {
        constexpr int kBatch = 8;
        const uint32_t per = (total + kThreads - 1u) / kThreads;
        uint32_t i = (uint32_t)tid * per;
        const uint32_t iend = min(total, i + per);
        uint32_t g = 0, gbase = 0, gend = 0;
        if (i < iend) {
            uint32_t lo_g = 0, hi_g = G - 1;                           // first slice whose prefix exceeds i
            while (lo_g < hi_g) {
                const uint32_t mid = (lo_g + hi_g) >> 1;
                if (t.take[mid] > i) hi_g = mid; else lo_g = mid + 1;
            }
            g = lo_g; gbase = g ? t.take[g - 1] : 0u; gend = t.take[g];
        }
        if (per == 1u) {                                               // a short list: one entry, no walking
            if (i < iend) {
                const uint64_t e = v.stash[((size_t)row * G + g) * kStashCap + (i - gbase)];
                uint32_t b = rebase_bits((uint32_t)(e >> 32), t.delta[g]);
                if (b < cutrow) b = 0;
                t.list[i] = ((uint64_t)b << 32) | (uint32_t)e;
            }
            i = iend;
        }
        while (i < iend) {
            uint64_t e[kBatch];
            uint32_t sl[kBatch];
            const uint32_t n = min((uint32_t)kBatch, iend - i);
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                e[u] = 0; sl[u] = 0;
                if ((uint32_t)u < n) {
                    while (i + (uint32_t)u >= gend) { ++g; gbase = gend; gend = t.take[g]; }    // slices that give nothing are skipped
                    e[u] = v.stash[((size_t)row * G + g) * kStashCap + (i + (uint32_t)u - gbase)];
                    sl[u] = g;
                }
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if ((uint32_t)u < n) {
                    uint32_t b = rebase_bits((uint32_t)(e[u] >> 32), t.delta[sl[u]]);
                    if (b < cutrow) b = 0;                             // plan B: below the complete part; 0 matches nothing
                    t.list[i + (uint32_t)u] = ((uint64_t)b << 32) | (uint32_t)e[u];
                }
            i += n;
        }
    }
    __syncthreads();
    uint32_t exb = f.bin >> 2;
    if (subset) {
        // level 1 again, on the gathered tokens alone
        for (int b = tid; b < kSB; b += kThreads) s.g[kBin0 + b] = 0;
        __syncthreads();
        for (uint32_t i = tid; i < total; i += kThreads) {
            const uint32_t b = (uint32_t)(t.list[i] >> 32);
            if (b) atomicAdd(reinterpret_cast<unsigned long long *>(&s.g[b >> 21]), (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
        }
        __syncthreads();
        f = hist_find_level1<false, true>(s, top_k, p.top_p, lane, wave);
        if (f.bin == 0u) {
            // even all of them are neither top_k tokens nor top_p of the mass
            if (tid == 0) {
                const uint32_t slot = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
                v.need[slot] = row;
            }
            return;
        }
        exb = f.bin >> 2;
    }

    // remaining digits of the threshold, on the gathered tokens
    uint32_t lo = f.bin << 21, span = (1u << 21) - 1u;
    for (uint32_t lv = 2; lv <= (uint32_t)kLevels && f.cnt_bin > 1u; ++lv) {
        const uint32_t dsh = level_shift(lv);
        lds_hist_zero(s, 128);
        __syncthreads();
        for (uint32_t i = tid; i < total; i += kThreads) {
            const uint32_t b = (uint32_t)(t.list[i] >> 32);
            if (b - lo <= span) lds_hist_add(s, (b >> dsh) & 127u, b);
        }
        __syncthreads();
        f = hist_find128(s, s.hm, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
        lo |= f.bin << dsh;
        span = (1u << dsh) - 1u;
    }
    if (span != 0u) {                                    // a single token left in the range: the threshold itself
        for (uint32_t i = tid; i < total; i += kThreads) {
            const uint32_t b = (uint32_t)(t.list[i] >> 32);
            if (b - lo <= span) s.bc32[6] = b;
        }
        __syncthreads();
        lo = s.bc32[6];
    }
    const uint32_t thr = lo;
    if (drawer) {                                        // the row is finished here: this draw is used up
        rng_st[2] = rs[2] + 1u;
        if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
    }
    if (tid == 0) {
        const Target tg = tie_and_target(p, row, p.inj_u ? 0ull : t.rand64, xmax, D, P, thr, f.cnt_above, f.cnt_bin, f.mass_above, 0u, true);   // rounds = 0: no cluster histogram
        s.bc64[1] = tg.w_tie; s.bc128[0] = tg.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    u128 r = s.bc128[0];
    auto weight = [&](uint32_t b) -> uint64_t { return (b > thr) ? w_of_bits(b) : (b == thr ? w_tie : 0); };

    // inverse CDF in index order: slice, then run of tokens, then token
    constexpr uint32_t sh_slice = SLICE_LOG2;
    constexpr uint32_t sh_run = sh_slice - 8;                                  // 256 runs of at most 64 tokens
    static_assert(SLICE_LOG2 >= 8 && SLICE_LOG2 <= 14, "runs must fit the final all-pairs step");
    constexpr uint32_t kPairs = 64;
    const uint64_t *cands = t.small;                                           // what the all-pairs step works on
    uint32_t nkept = total;
    if (total <= kPairs) cands = t.list;                                       // the whole list is few enough as it is
    else {
    const uint32_t ga = bucket_step(s, t, total, sh_slice, 0u, 0xFFFFFFFFu, r, weight, lane, wave);
    uint32_t lo_b = ga << sh_slice, len_b = 1u << sh_slice;
    // the kept tokens of that slice: few enough for the all-pairs step as they are, as a rule;
    // otherwise the slice is narrowed to one of its 256 runs first
    auto collect = [&]() {
        if (tid == 0) t.nsmall = 0;
        __syncthreads();
        for (uint32_t i = tid; i < total; i += kThreads) {
            const uint64_t e = t.list[i];
            const uint32_t idx = (uint32_t)e;
            if (idx - lo_b < len_b && weight((uint32_t)(e >> 32))) {
                const uint32_t o = atomicAdd(&t.nsmall, 1u);
                if (o < kPairs) t.small[o] = e;
            }
        }
        __syncthreads();
        return t.nsmall;
    };
    nkept = collect();
    if (nkept > kPairs) {
        __syncthreads();                                                       // everyone has read the count
        const uint32_t gb = bucket_step(s, t, total, sh_run, lo_b, lo_b + len_b, r, weight, lane, wave);
        lo_b += gb << sh_run; len_b = 1u << sh_run;
        nkept = collect();
    }
    }
    // all pairs: every kept token of the range adds up the weights at or before it in index order;
    // the four waves take a quarter of the addends each
    static_assert(kWaves == 4 && offsetof(Lds, cand) % 16 == 0 && sizeof(s.cand) >= 64 * 16 + 4 * 64 * 16, "records and partial sums live in s.cand");
    const uint32_t ns = min(nkept, kPairs);
    uint4 *rec = reinterpret_cast<uint4 *>(s.cand);                             // weight (x, y), index (z)
    u128 *partial = reinterpret_cast<u128 *>(s.cand) + kPairs;
    uint64_t me = 0, wme = 0;
    if ((uint32_t)tid < ns) {
        me = cands[tid];
        wme = weight((uint32_t)(me >> 32));
        rec[tid] = make_uint4((uint32_t)wme, (uint32_t)(wme >> 32), (uint32_t)me, 0u);
    }
    __syncthreads();
    {
        const uint32_t per = (ns + 3u) >> 2, j0 = (uint32_t)wave * per, j1 = min(ns, j0 + per);
        const uint32_t mine = (uint32_t)lane < ns ? rec[lane].z : 0u;
        uint64_t lo32 = 0, hi32 = 0;                                              // halves summed apart: no carries
#pragma unroll 4
        for (uint32_t j = j0; j < j1; ++j) {
            const uint4 o = rec[j];
            const bool c = o.z <= mine;
            lo32 += c ? o.x : 0u;
            hi32 += c ? o.y : 0u;
        }
        partial[wave * (int)kPairs + lane] = (u128)lo32 + ((u128)hi32 << 32);
    }
    __syncthreads();
    if ((uint32_t)tid < ns) {
        const u128 upto = partial[tid] + partial[kPairs + tid] + partial[2 * kPairs + tid] + partial[3 * kPairs + tid];
        if (upto - wme < r && r <= upto) {
            p.out[row] = (int32_t)(uint32_t)me;
            if (p.diag) p.diag[row].index = (int32_t)(uint32_t)me;
        }
    }
}

template <int SLICE_LOG2>
__global__ void __launch_bounds__(kThreads) finish_kernel(const Params p, const StreamView v)
{
    __shared__ Lds s;
    __shared__ LdsB t;
    extern __shared__ __align__(16) unsigned char finish_dyn[];
    t.list = reinterpret_cast<uint64_t *>(finish_dyn);       // every thread writes the same value
    finish_row<SLICE_LOG2>(p, v, s, t, blockIdx.x);
}

// Launch-plus-one-read floor: same grid, each row read once, one int out.
template <int R>
__global__ void __launch_bounds__(kThreads) floor_kernel(const float *logits, int64_t row_stride, int32_t *out,
                                                         int32_t V, uint32_t G)
{
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const uint32_t V4 = (uint32_t)V >> 2;
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + threadIdx.x;
    const float4 *lg = reinterpret_cast<const float4 *>(logits + (int64_t)row * row_stride);
    float m = -3.402823466e+38f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const float4 v = lg[min(base4 + (uint32_t)(j * kThreads), V4 - 1)];
        m = fmaxf(m, fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
    }
    uint32_t k = wave_max_u32(fkey(m));
    if ((threadIdx.x & 63) == 0) atomicMax(reinterpret_cast<uint32_t *>(out + row), k);
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

// What a call reads before it writes: the launch header and its row records.
__global__ void __launch_bounds__(256) clear_records_kernel(uint4 *hdr, uint4 *recs, size_t n16)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) recs[i] = make_uint4(0u, 0u, 0u, 0u);
    if (blockIdx.x == 0 && threadIdx.x < sizeof(WsHeader) / 16) hdr[threadIdx.x] = make_uint4(0u, 0u, 0u, 0u);
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
        const int R = force_r;
        if ((R == 1 || R == 2 || R == 4 || R == 8 || R == 16 || R == 32) && R <= maxR && parts(R) <= (uint32_t)kMaxParts)
            return {R, parts(R)};
    }
    // Measured on MI355X: a cluster works best with at most ~64 workgroups (each exchange costs
    // more the more peers poll), slices of 32 float4 per thread only pay for rows of a quarter
    // million tokens and more (the variant spills), and a call wants a few hundred workgroups in
    // flight -- 256 for small batches, where latency counts, 512 beyond.
    int minR = maxR;
    for (int R = 1; R <= maxR; R *= 2)
        if (parts(R) <= 64u) { minR = R; break; }
    const int topR = (V4 >= 65536u || minR > 16) ? maxR : (maxR < 16 ? maxR : 16);
    const uint64_t want = B <= 16 ? 256 : 512;
    for (int R = topR; R >= minR; R /= 2)
        if ((uint64_t)B * parts(R) >= want) return {R, parts(R)};
    return {minR, parts(minR)};
}


// Streaming geometry: workgroups of 256 threads; slices of 16384 tokens (16 float4 per thread), or
// of 4096 tokens (4 float4) for calls of up to kStreamSmall tokens in rows of up to 262144, where a
// shorter slice shortens the one wave of workgroups the whole pass consists of (longer rows would
// be cut into more slices than a finishing workgroup handles quickly).
constexpr int kStreamNT = 256;
constexpr uint64_t kStreamSmall = 1ull << 22;
constexpr uint32_t kListGrid = 256;            // workgroups of the launch for the rows handed on (they loop)
static int stream_r(int32_t B, int32_t V) { return (uint64_t)B * (uint64_t)V <= kStreamSmall && V <= 262144 ? 4 : 16; }
static uint32_t stream_parts(int32_t V, int R) { return ((uint32_t)V / 4 + kStreamNT * R - 1) / (kStreamNT * R); }
static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
struct StreamLayout { size_t hdr, cum, shist, stash, need, end; };
static StreamLayout stream_layout(int32_t B, size_t parts, size_t base)
{
    StreamLayout l;
    l.hdr = align256(base);
    l.cum = align256(l.hdr + parts * sizeof(PartHdr));
    l.shist = align256(l.cum + parts * kSB * sizeof(uint32_t));
    l.stash = align256(l.shist + parts * kSB * sizeof(uint64_t));
    l.need = align256(l.stash + parts * kStashCap * sizeof(uint64_t));
    l.end = align256(l.need + (size_t)B * sizeof(uint32_t));
    return l;
}
// Bytes of per-slice data a workspace for (B, V) sets aside: enough for the long slices of (B, V)
// itself and for the short slices of any call of at most B rows that takes them (at most
// kStreamSmall tokens: fewer than kStreamSmall / 4096 + B slices), so that the size grows with
// B and with V and a workspace for the largest B and V serves every smaller call.
static size_t stream_bytes(int32_t B, int32_t V)
{
    const size_t longs = stream_layout(B, (size_t)B * stream_parts(V, 16), sizeof(WsHeader)).end;
    size_t small_parts = (size_t)B * stream_parts(V, 4);
    const size_t cap = (size_t)(kStreamSmall / 4096) + (size_t)B;
    if (small_parts > cap) small_parts = cap;
    const size_t shorts = stream_layout(B, small_parts, sizeof(WsHeader)).end;
    return longs > shorts ? longs : shorts;
}

}  // namespace rs

// The caller's routing state (see rapid_sampling.h).  word[0], word[1]: "most rows were handed on"
// as last reported by a streaming call with / without a bounding top_k; word[2]: RS_ERR_DEVICE
// once a kernel gave up a wait.  calls[]: calls routed away from the streaming path since.
struct rs_policy {
    int32_t *word;
    uint32_t calls[2];
};

namespace rs {

// The streaming path works when the kept set is small next to the row; a row for which it does
// not is handed to the cluster kernel in a third launch, and a call whose rows mostly end that way
// has wasted a pass.  With a bounding top_k that takes unusual rows (ties of thousands of tokens);
// without one (nucleus sampling alone) it is simply a flat distribution, so such a call is an
// attempt.  The launch for the rows handed on reports "most of them: yes/no" into a word of the
// caller's rs_policy, one word for calls with a bounding top_k and one for calls without, and
// this function looks at the word -- without waiting for anything; a stale value only delays the
// switch -- before it chooses the path of the next call: after a call that handed most rows on,
// calls of that kind go straight to the cluster kernel and one in 64 streams again.  Without a
// policy, calls with a bounding top_k always stream and calls without never do.
//
// Measured on MI355X, back to back: with a bounding top_k the streaming path beats the cluster
// kernel from 131072 tokens per call upwards (15-17 us for small calls against 16-31 us, 2-3
// times faster for large ones); below that the single launch wins by up to a microsecond.
enum { kPathCluster = 0, kPathStream = 1, kPathAttempt = 2 };
static int choose_path(int32_t B, int32_t V, int32_t top_k, float top_p, bool pen, const rs_options *opt)
{
    if (pen) return kPathCluster;
    const bool bounded = top_k <= kStreamK;
    const int force = opt ? opt->path : RS_PATH_AUTO;
    if (force == RS_PATH_CLUSTER) return kPathCluster;
    if (force == RS_PATH_STREAM) return bounded ? kPathStream : kPathCluster;
    if (force == RS_PATH_ATTEMPT) return bounded ? kPathStream : kPathAttempt;
    if ((uint64_t)B * (uint64_t)V < (1ull << 17)) return kPathCluster;
    if (!bounded && !(top_p < 1.0f)) return kPathCluster;      // everything is kept: nothing a stash could hold
    rs_policy *pol = opt ? opt->policy : nullptr;
    if (!pol) return bounded ? kPathStream : kPathCluster;
    const int yes = bounded ? kPathStream : kPathAttempt, kind = bounded ? 0 : 1;
    const bool failing = *(volatile int32_t *)(pol->word + kind) != 0;
    return (!failing || (++pol->calls[kind] & 63u) == 0u) ? yes : kPathCluster;
}

template <bool PEN>
static hipError_t launch_sample(int R, dim3 grid, hipStream_t st, const Params &p)
{
    switch (R) {
    case 1:  hipLaunchKernelGGL((sample_kernel<1, PEN>),  grid, dim3(kThreads), 0, st, p); break;
    case 2:  hipLaunchKernelGGL((sample_kernel<2, PEN>),  grid, dim3(kThreads), 0, st, p); break;
    case 4:  hipLaunchKernelGGL((sample_kernel<4, PEN>),  grid, dim3(kThreads), 0, st, p); break;
    case 8:  hipLaunchKernelGGL((sample_kernel<8, PEN>),  grid, dim3(kThreads), 0, st, p); break;
    case 16: hipLaunchKernelGGL((sample_kernel<16, PEN>), grid, dim3(kThreads), 0, st, p); break;
    default:
        if constexpr (!PEN) hipLaunchKernelGGL((sample_kernel<32, false>), grid, dim3(kThreads), 0, st, p);
        break;
    }
    return hipGetLastError();
}

static hipError_t launch_list(int R, dim3 grid, hipStream_t st, const Params &p, bool once)
{
    if (once) {
        switch (R) {
        case 1:  hipLaunchKernelGGL((sample_list_once_kernel<1>),  grid, dim3(kThreads), 0, st, p); break;
        case 2:  hipLaunchKernelGGL((sample_list_once_kernel<2>),  grid, dim3(kThreads), 0, st, p); break;
        case 4:  hipLaunchKernelGGL((sample_list_once_kernel<4>),  grid, dim3(kThreads), 0, st, p); break;
        case 8:  hipLaunchKernelGGL((sample_list_once_kernel<8>),  grid, dim3(kThreads), 0, st, p); break;
        case 16: hipLaunchKernelGGL((sample_list_once_kernel<16>), grid, dim3(kThreads), 0, st, p); break;
        default: hipLaunchKernelGGL((sample_list_once_kernel<32>), grid, dim3(kThreads), 0, st, p); break;
        }
        return hipGetLastError();
    }
    switch (R) {
    case 1:  hipLaunchKernelGGL((sample_list_kernel<1>),  grid, dim3(kThreads), 0, st, p); break;
    case 2:  hipLaunchKernelGGL((sample_list_kernel<2>),  grid, dim3(kThreads), 0, st, p); break;
    case 4:  hipLaunchKernelGGL((sample_list_kernel<4>),  grid, dim3(kThreads), 0, st, p); break;
    case 8:  hipLaunchKernelGGL((sample_list_kernel<8>),  grid, dim3(kThreads), 0, st, p); break;
    case 16: hipLaunchKernelGGL((sample_list_kernel<16>), grid, dim3(kThreads), 0, st, p); break;
    default: hipLaunchKernelGGL((sample_list_kernel<32>), grid, dim3(kThreads), 0, st, p); break;
    }
    return hipGetLastError();
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

int rs_version(void) { return 400; }

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
    *bytes = stream_bytes(B, V) + (size_t)B * sizeof(RowCtl);
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

int rs_policy_create(rs_policy **out)
{
    if (!out) return RS_ERR_NULL;
    *out = nullptr;
    rs_policy *pol = new (std::nothrow) rs_policy;
    if (!pol) return RS_ERR_LAUNCH;
    pol->word = nullptr; pol->calls[0] = 0; pol->calls[1] = 0;
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
    *state = (w[1] != 0 ? 1 : 0) | (w[0] != 0 ? 2 : 0);
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

int rs_sample_ex(const void *logits, int32_t logits_dtype, int64_t row_stride, float *penalties, int32_t *out,
                 void *rng_state, const float *injected_u, int32_t B, int32_t V,
                 float presence, float repetition, float decay,
                 float log2e_inv_temp, int32_t top_k, float top_p,
                 void *workspace, size_t workspace_bytes,
                 rs_row_diag *diag, uint32_t *e_bits, const rs_options *opt, void *stream)
{
    if (!logits || !out || !workspace || (!rng_state && !injected_u)) return RS_ERR_NULL;
    if (logits_dtype != RS_DTYPE_F32 && logits_dtype != RS_DTYPE_BF16 && logits_dtype != RS_DTYPE_F16) return RS_ERR_ARG;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    if (!(top_k >= 1 && top_k <= V) || !(top_p > 0.0f && top_p <= 1.0f) || !(log2e_inv_temp > 0.0f)) return RS_ERR_ARG;
    if (opt && (opt->path < RS_PATH_AUTO || opt->path > RS_PATH_ATTEMPT || opt->slice_r < 0)) return RS_ERR_ARG;
    if (((uintptr_t)logits & (logits_dtype == RS_DTYPE_F32 ? 15 : 7)) || (B > 1 && (row_stride & 3)) || ((uintptr_t)penalties & 15) || ((uintptr_t)e_bits & 15))
        return RS_ERR_ALIGN;
    size_t need = 0;
    rs_workspace_bytes(B, V, &need);
    if (workspace_bytes < need || ((uintptr_t)workspace & 255)) return RS_ERR_WORKSPACE;

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
    p.need = nullptr; p.stash_k = (uint32_t)top_k; p.report = 0;
    p.host_words = opt && opt->policy ? opt->policy->word : nullptr;
    dim3 grid((uint32_t)B * g.G);
    const int path = choose_path(B, V, top_k, top_p, pen, opt);
    if (path != kPathCluster) {
        const int sr = stream_r(B, V);
        StreamView v;
        v.G = stream_parts(V, sr);
        const StreamLayout l = stream_layout(B, (size_t)B * v.G, sizeof(WsHeader));
        char *w = (char *)workspace;
        v.hdr = (PartHdr *)(w + l.hdr); v.stash = (uint64_t *)(w + l.stash); v.cum = (uint32_t *)(w + l.cum);
        v.shist = (uint64_t *)(w + l.shist);
        v.need = (uint32_t *)(w + l.need);
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
        p.report = path == kPathAttempt ? 1u : 0u;
        const size_t dyn = (size_t)v.list_cap * sizeof(uint64_t);
        const dim3 sgrid((uint32_t)B * v.G), sblock(kStreamNT);
        if (sr == 4) {
            if (logits_dtype == RS_DTYPE_F32) hipLaunchKernelGGL((stream_kernel<4, kStreamNT, RS_DTYPE_F32>), sgrid, sblock, 0, st, p, v);
            else if (logits_dtype == RS_DTYPE_BF16) hipLaunchKernelGGL((stream_kernel<4, kStreamNT, RS_DTYPE_BF16>), sgrid, sblock, 0, st, p, v);
            else hipLaunchKernelGGL((stream_kernel<4, kStreamNT, RS_DTYPE_F16>), sgrid, sblock, 0, st, p, v);
            hipLaunchKernelGGL((finish_kernel<12>), dim3((uint32_t)B), dim3(kThreads), dyn, st, p, v);
        } else {
            if (logits_dtype == RS_DTYPE_F32) hipLaunchKernelGGL((stream_kernel<16, kStreamNT, RS_DTYPE_F32>), sgrid, sblock, 0, st, p, v);
            else if (logits_dtype == RS_DTYPE_BF16) hipLaunchKernelGGL((stream_kernel<16, kStreamNT, RS_DTYPE_BF16>), sgrid, sblock, 0, st, p, v);
            else hipLaunchKernelGGL((stream_kernel<16, kStreamNT, RS_DTYPE_F16>), sgrid, sblock, 0, st, p, v);
            hipLaunchKernelGGL((finish_kernel<14>), dim3((uint32_t)B), dim3(kThreads), dyn, st, p, v);
        }
        if (hipGetLastError() != hipSuccess) return RS_ERR_LAUNCH;
        p.need = v.need;               // the cluster kernel follows for the rows the finish left over
        // Workgroups for the rows handed on.  Few rows are expected when top_k bounds the kept set: a
        // small grid whose workgroups take tickets until the list is exhausted.  After an attempt it
        // may be all of them: one workgroup per slice of every row, as in the cluster kernel; those
        // beyond the list leave at once.
        if (path == kPathStream && grid.x > kListGrid) grid.x = kListGrid / g.G * g.G > 0 ? kListGrid / g.G * g.G : g.G;
    }
    const hipError_t e = p.need ? launch_list(g.R, grid, (hipStream_t)stream, p, path == kPathAttempt)
                       : pen ? launch_sample<true>(g.R, grid, (hipStream_t)stream, p)
                             : launch_sample<false>(g.R, grid, (hipStream_t)stream, p);
    return e == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

int rs_sample_static(const void *logits, int32_t logits_dtype, int64_t row_stride, float *penalties, int32_t *out,
                     void *rng_state, const float *injected_u, int32_t B, int32_t V,
                     float presence, float repetition, float decay,
                     float log2e_inv_temp, int32_t top_k, float top_p,
                     rs_row_diag *diag, uint32_t *e_bits, const rs_options *opt, void *stream)
{
    size_t need = 0;
    const int rc = rs_workspace_bytes(B, V, &need);
    if (rc != RS_OK) return rc;
    if (need > (size_t)RS_STATIC_SCRATCH_BYTES) return RS_ERR_SCRATCH;
    // every GPU holds its own copy of the array at its own address: looked up once per device
    constexpr int kMaxDevices = 64;
    static std::atomic<void *> base[kMaxDevices];
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return RS_ERR_LAUNCH;
    void *ws = base[dev].load(std::memory_order_acquire);
    if (!ws) {
        if (hipGetSymbolAddress(&ws, HIP_SYMBOL(scratch)) != hipSuccess || !ws) return RS_ERR_LAUNCH;
        base[dev].store(ws, std::memory_order_release);
    }
    // The array keeps what the last call left.  A call leaves it clean unless a wait gave up; the launch
    // header and this call's row records are cleared all the same, by a kernel (not a memset node: the
    // call may be under capture), so that every call starts from zero whatever came before.
    const size_t rec_bytes = (size_t)B * sizeof(RowCtl);
    char *recs = (char *)ws + (size_t)RS_STATIC_SCRATCH_BYTES - rec_bytes;
    const size_t n16 = rec_bytes / 16;
    const uint32_t blocks = (uint32_t)(n16 / 1024 < 1 ? 1 : n16 / 1024 > 1024 ? 1024 : n16 / 1024);
    hipLaunchKernelGGL(clear_records_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint4 *)ws, (uint4 *)recs, n16);
    if (hipGetLastError() != hipSuccess) return RS_ERR_LAUNCH;
    return rs_sample_ex(logits, logits_dtype, row_stride, penalties, out, rng_state, injected_u, B, V, presence,
                        repetition, decay, log2e_inv_temp, top_k, top_p, ws, (size_t)RS_STATIC_SCRATCH_BYTES, diag,
                        e_bits, opt, stream);
}

int rs_floor_read(const float *logits, int64_t row_stride, int32_t *out, int32_t B, int32_t V, void *stream)
{
    if (!logits || !out) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    const Geometry g = choose_geometry(B, V, false, 0);
    const dim3 grid((uint32_t)B * g.G);
    hipStream_t st = (hipStream_t)stream;
    switch (g.R) {
    case 1:  hipLaunchKernelGGL((floor_kernel<1>),  grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    case 2:  hipLaunchKernelGGL((floor_kernel<2>),  grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    case 4:  hipLaunchKernelGGL((floor_kernel<4>),  grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    case 8:  hipLaunchKernelGGL((floor_kernel<8>),  grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    case 16: hipLaunchKernelGGL((floor_kernel<16>), grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    default: hipLaunchKernelGGL((floor_kernel<32>), grid, dim3(kThreads), 0, st, logits, row_stride, out, V, g.G); break;
    }
    return hipGetLastError() == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

}  // extern "C"
