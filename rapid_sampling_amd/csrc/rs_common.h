// Shared declarations of the MI355X token sampler's kernels: workspace records, launch
// parameters, histogram packing, workgroup-level reductions and scans, the exchanges between
// the workgroups of a row.  Device code only (included by the .hip files of this directory).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "rapid_sampling.h"
#include "rs_device.h"

namespace rs {


constexpr int      kThreads   = 256;          // 4 waves, one per SIMD
constexpr int      kWaves     = kThreads / kWave;
constexpr int      kMaxParts  = 256;          // workgroups per row, at most
constexpr int      kNB        = 512;          // bins per histogram: level 1 uses 164, deeper levels 128
constexpr int      kLevels    = 4;            // 10 + 7 + 7 + 7 bits
constexpr int      kCap       = 1024;         // tokens of a boundary bin that are gathered
constexpr uint64_t kSpinLimit = 200000000ull; // 2 s of the 100 MHz wall clock

constexpr uint64_t kValid     = 1ull << 63;   // marks a written exchange word
constexpr uint32_t kVerdictFallback = 0xFFFFFFFFu;   // the finishing workgroup could not finish the row from the stashes

struct alignas(256) WsHeader {
    uint32_t unused0;
    uint32_t finished;    // workgroups that have left the running launch
    int32_t  error;       // sticky RS_ERR_DEVICE
    uint32_t n_need;      // rows of the running (or last) streaming call that the finishing workgroups did the slow way
    uint32_t spin_ticks;  // bound of a wait in units of 1024 wall-clock ticks; 0 = the default (2 s)
    uint32_t last_call;   // 1 | word << 8 after a streaming call that no later call has reported on yet (word: the report word of the caller's policy the call writes, Params::report), else 0
    uint32_t gave_up[4];  // the first wait that gave up since the workspace was set up: site, row << 16 | slice, what it had, what it waited for
    uint32_t pad[54];
    // Logical workgroup ids of a launch larger than the device holds at once: eight counters, one per
    // workgroup id modulo 8, each on a cache line of its own (take_ticket).
    uint32_t ticket[8][64];
};
static_assert(sizeof(WsHeader) == 2304, "tests that spoil a workspace leave its header alone: tests/capi.py HEADER_BYTES");


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
    uint32_t arrived;     // one-launch path: workgroups of the row that have published their slice
    uint32_t verdict;     // one-launch path: 0 pending, sampled token + 1, or kVerdictFallback
    uint32_t pad[3];
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
    int32_t      dtype;        // RS_DTYPE_* of the logits
    uint32_t     report;       // index of the report word of the caller's policy a streaming call writes (4..12: kind of call x size class), 0 none
    uint32_t     attempt;      // the call has no bounding top_k: its streaming pass is an attempt
    uint32_t     tell_lists;   // streaming finish: a row whose list is long enough for another kernel to be faster says so to the policy
    uint32_t     probe;        // wide path as a probe for the streaming path: rows whose kept set the stashes would not hold are reported as slow
    int32_t     *host_words;   // the caller's rs_policy: pinned host memory, [2] error, [4..12] routing reports; or null
    int32_t      defer_pen;    // penalties enter x and are not rewritten from the registers at the end: 1 a later pass over them
                               // applies decay and one-hot add; 2 the streaming pass writes the decayed values itself and notes
                               // the old non-zero ones, the finish patches the sampled token (see stream_pen_kernel)
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

// Logical id of this workgroup in a launch larger than the device holds at once: ids follow the order
// in which workgroups start.  One counter for the whole launch would be a few thousand fetch-adds on
// one word, served at about 12 ns each whatever else the memory system does (a launch of 1024
// workgroups: 13 us until the last one has its id; of 4096: 48 us); eight counters on cache lines of
// their own, chosen by the hardware's workgroup id modulo 8, are served side by side (3 and 8 us).
// Class c hands out the ids congruent to c modulo 8, in the order its workgroups start, and there
// are exactly as many workgroups in a class as ids of that residue below the launch size, so every
// id is taken once.  The hardware binds workgroup b to XCD b mod 8, so an XCD's workgroups draw from
// one counter and hold, at any time, the lowest ids of their class not yet finished: the earliest
// unfinished row has all its workgroups running or next to start on every XCD.
__device__ __forceinline__ uint32_t take_ticket(WsHeader *hdr)
{
    const uint32_t c = blockIdx.x & 7u;
    const uint32_t mine = (gridDim.x - c + 7u) >> 3;     // workgroups of this class in the launch
    const uint32_t n = __hip_atomic_fetch_add(&hdr->ticket[c][0], 1u, __ATOMIC_RELAXED, RS_AGENT);
    // every workgroup takes exactly one: after the class's last the counter is not touched again,
    // and is put back for the next call
    if (n == mine - 1u) a_store(&hdr->ticket[c][0], 0u);
    return n * 8u + c;
}

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
// Loads of data that is read exactly once (the logits): marked non-temporal, so that the lines are
// not kept in the caches at the expense of what is re-read.  On MI355X a pass over 512 MiB reads at
// 6.8-7.0 TB/s this way against 6.1-6.3 TB/s with plain loads.
typedef uint32_t rs_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t rs_u32x2 __attribute__((ext_vector_type(2)));
#ifndef RS_NT
#define RS_NT 1
#endif
__device__ __forceinline__ uint4 load_once(const uint4 *p)
{
    if (!RS_NT) return *p;
    const rs_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const rs_u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_once(const uint2 *p)
{
    const rs_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const rs_u32x2 *>(p));
    return make_uint2(v.x, v.y);
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
    uint32_t who, seen, want; // for the same: row << 16 | slice of this workgroup; what its current wait has and waits for
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
__device__ __forceinline__ void give_up(Lds &s, WsHeader *hdr, uint32_t site);

// Bounded wait bookkeeping: thread 0 looks at the wall clock now and then; the
// verdict is read by everyone after a workgroup barrier, so it is uniform.
struct SpinGuard {
    uint64_t t0;
    uint32_t spins;
    __device__ __forceinline__ void start() { t0 = (uint64_t)wall_clock64(); spins = 0; }
    // call by every thread once per polling round, before the round's __syncthreads
    __device__ __forceinline__ void tick(Lds &s, WsHeader *hdr, uint32_t site)
    {
        if (threadIdx.x == 0 && (++spins & 255u) == 0 && (uint64_t)wall_clock64() - t0 > spin_limit(hdr)) give_up(s, hdr, site);
    }
};

// Sites of the waits: 1 a histogram level of the cluster, 2 its level 1, 3 the gathered tokens, 4 the
// kept masses, 5 the sampled index, 6 the verdict of the one-launch path.
__device__ __forceinline__ void give_up(Lds &s, WsHeader *hdr, uint32_t site)
{
    uint32_t none = 0u;
    if (__hip_atomic_compare_exchange_strong(&hdr->gave_up[0], &none, site, __ATOMIC_RELAXED, __ATOMIC_RELAXED, RS_AGENT)) {
        a_store(&hdr->gave_up[1], s.who); a_store(&hdr->gave_up[2], s.seen); a_store(&hdr->gave_up[3], s.want);
    }
    a_store(&hdr->error, (int32_t)RS_ERR_DEVICE);
    if (s.host_words) __hip_atomic_store(s.host_words + 2, (int32_t)RS_ERR_DEVICE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    s.abort = 1;
}

// Routing report of the streaming path.  A row that the finishing workgroup has to do the slow way
// (alone, from the logits, in several passes) costs several times what the general kernel takes for
// the whole call, so one such row is reason enough to send the next calls of that kind to the
// general kernel.  Slow rows are counted in the workspace header and the first of a call sets the
// word of the caller's policy at once (finish_row); that a call went WELL is said by the first
// thread of the next call on the workspace, streaming or not, which collects the count (its memory
// round trip overlaps with the thread's loads of the logits) and clears the word.
struct PrevCall { uint32_t slow_rows, meta; };
__device__ __forceinline__ PrevCall report_begin(const Params &p)
{
    PrevCall pc;
    pc.slow_rows = __hip_atomic_exchange(&p.hdr->n_need, 0u, __ATOMIC_RELAXED, RS_AGENT);
    pc.meta = a_load(&p.hdr->last_call);                 // 1 | word << 8 of a streaming call not yet reported on, else 0
    return pc;
}
// `streaming`: the reporting call is a streaming call itself, to be reported on by the next one
__device__ __forceinline__ void report_end(const Params &p, const PrevCall &pc, const bool streaming)
{
    if (streaming) a_store(&p.hdr->last_call, 1u | (p.report << 8));
    else if (pc.meta) a_store(&p.hdr->last_call, 0u);
    if (p.host_words && pc.meta)
        __hip_atomic_store(p.host_words + ((pc.meta >> 8) & 15u), pc.slow_rows ? 1 : 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
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
        guard.tick(s, hdr, 1u);
        const uint32_t total = block_sum_u32(s, c, lane, wave);
        if (total == expected) return true;
        if (s.abort) return false;
        if (threadIdx.x == 0) { s.seen = total; s.want = expected; }
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
        guard.tick(s, hdr, 2u);
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
        if (tid == 0) { s.seen = total; s.want = expected; }
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
template <bool LOCAL, bool GIVEN_P = false, typename L = Lds>
__device__ __forceinline__ Found hist_find_level1(L &s, uint64_t top_k, float top_p, int lane, int wave)
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
            if constexpr (LOCAL) {
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
template <typename L = Lds>
__device__ __forceinline__ Found hist_find128(L &s, const uint64_t *arr, uint32_t cnt0, u128 mass0,
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


// Float4 groups per thread of the streaming pass's long slices (slices of 1024 * kStreamLongR tokens)
#ifndef RS_STREAM_R
#define RS_STREAM_R 16
#endif
constexpr int kStreamLongR = RS_STREAM_R;
constexpr int kStreamLongLog2 = kStreamLongR == 16 ? 14 : kStreamLongR == 8 ? 13 : 12;

// ---- per-slice records of the streaming path (laid out in the workspace by the host) ----
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

// A slice's note of its penalties (stream_pen_kernel): word 0 = count, or kPenDeferred when the slice left its
// penalties untouched; then count entries (old value's bits << 32 | token index in the row), the penalties
// whose bit pattern was not +0.0 before the call.
constexpr int      kPenCap      = 512;        // words per slice: 511 non-zero penalties among 16384 tokens, 3.1 %
constexpr int      kPenWave     = 160;        // of which one wave (4096 tokens) can note this many
constexpr uint64_t kPenDeferred = 1ull << 63;

struct StreamView {
    PartHdr  *hdr;        // [B][G]
    uint64_t *pens;       // [B][G][kPenCap]   penalties at scale only, else null
    uint64_t *stash;      // [B][G][kStashCap]   bits(e, slice frame) << 32 | index, by descending bin
    uint32_t *cum;        // [B][G][kSB]   tokens of the slice in this bin and the bins above it
    uint64_t *shist;      // [B][G][kSB]   the slice's own bins (slice frame), as it added them to the row's
    uint32_t  G;          // slices per row
    uint32_t  list_cap;   // entries of the finishing workgroup's token list (a power of two up to kFinCap)
};


// Launchers, one per translation unit that instantiates the kernels.
hipError_t launch_sample(bool pen, int R, dim3 grid, hipStream_t st, const Params &p);
hipError_t launch_stream_pen(uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v);
hipError_t launch_penalty_fix(hipStream_t st, const Params &p, const StreamView &v);
hipError_t launch_stream(int slice_r, int32_t dtype, bool keep, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p,
                         const StreamView &v);
hipError_t launch_fused(int slice_r, bool pen, uint32_t B, hipStream_t st, const Params &p, const StreamView &v);
hipError_t launch_wide(int slice_r, int32_t dtype, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v);
hipError_t launch_wide1(int slice_r, int32_t dtype, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v);
constexpr int32_t kRowMaxV = 65536;                      // the longest row the row kernel holds in its registers
hipError_t launch_row(int32_t dtype, uint32_t B, hipStream_t st, const Params &p);

}  // namespace rs
