// The streaming path: one wait-free pass over the logits, a finishing workgroup per row.
#pragma once

#include "rs_common.h"
#include "rs_cluster.h"

namespace rs {

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
//                   nucleus of thousands of tokens) it does alone, from the
//                   logits (finish_row_slow).
// A call that keeps every live token (top_k = V, top_p = 1) runs both kernels as a variant (KEEP):
// the pass stops behind the histogram and leaves each slice's mass, the finishing workgroup picks
// the slice from the masses and reads that one slice again (keep_pick).
// Lanes of a wave that add to one LDS address are served one after the other, and rows often put
// most of their tokens into a few bins.  So each bin is kept in kRep copies (lane l adds to copy
// l % kRep), and e is not clamped before it is counted: the histogram spans all 512 values of
// bits >> 21, the dead tokens (below 2^-40, often most of a row) spread over the bins below
// kBin0 by their own exponents, where nobody looks at them again.  The histogram is done with
// before the candidates are staged, and shares their memory.
// Eight copies for long slices; four for the middle ones, which keeps their histogram smaller than
// the candidate staging it shares memory with (six workgroups per CU); two for the short slices of
// small calls, where clearing and folding the copies would cost more than the few tokens of a thread.
template <int R> constexpr int stream_copies() { return R > 8 ? 8 : R == 8 ? 4 : 2; }
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

#ifndef RS_STREAM_WAVES
#define RS_STREAM_WAVES 3
#endif
// Stores of per-slice data: plain for the streaming path of separate launches (the kernel boundary makes
// them visible), device-scope atomic stores for the one-launch path, whose finishing workgroup
// reads them while the kernel is still running.
template <bool FUSED, typename T> __device__ __forceinline__ void put(T *p, T v)
{
    if (FUSED) a_store(p, v); else *p = v;
}
template <bool FUSED, typename T> __device__ __forceinline__ T get(const T *p)
{
    if (FUSED) return a_load(p); else return *p;
}

// One slice of the streaming pass, from the scaled logits in the registers (eb: x of this thread's
// 4R tokens, lmax their maximum) to its published record: the slice's frame, e in that frame (left
// in eb), the packed histogram added to the row's and kept under the slice's own name, cumulative
// counts, and the stash of its largest tokens with the value down to which it is complete.
// Returns the key of the slice's maximum.
template <int R, int NT, int kRep, bool FUSED, bool KEEP = false>     // KEEP: a call that keeps every live token (top_k = V, top_p = 1)
__device__ __forceinline__ uint32_t slice_count_and_stash(const Params &p, const StreamView &v, LdsA<kRep> &s, uint32_t (&eb)[R * 4],
                                                          const float lmax, const uint32_t row, const uint32_t part,
                                                          const uint32_t base4, const int nv)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    {
        uint4 *z = reinterpret_cast<uint4 *>(s.hm);                              // two bins per store
#pragma unroll
        for (int i = 0; i < kNB * kRep / 2 / NT; ++i) z[tid + i * NT] = make_uint4(0u, 0u, 0u, 0u);
        static_assert(kNB * kRep % (2 * NT) == 0, "whole stores");
    }
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
            if (j < nv) {
                if (FUSED) {
                    uint32_t *w = reinterpret_cast<uint32_t *>(&dst[base4 + j * NT]);
                    a_store(&w[0], eb[j * 4]); a_store(&w[1], eb[j * 4 + 1]); a_store(&w[2], eb[j * 4 + 2]); a_store(&w[3], eb[j * 4 + 3]);
                } else dst[base4 + j * NT] = make_uint4(eb[j * 4], eb[j * 4 + 1], eb[j * 4 + 2], eb[j * 4 + 3]);
            }
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
        put<FUSED>(&v.shist[((size_t)row * G + part) * kSB + tid], w);          // kept for rows whose slices lie far apart
        uint64_t *rowbins = FUSED ? (p.ctl_end - 1 - row)->h[0] : (p.ctl_end - 1 - row)->rowhist;
        if (w) a_add(&rowbins[((uint32_t)(int)mm * 4u + (uint32_t)tid - 160u) & 511u], w);
    }
    if constexpr (KEEP) {
        // every live token is kept: the bins and their mass (in this slice's frame, left where the
        // stash would begin) are all the finishing workgroup needs of this slice
        if (wave == 0) {
            u128 ms = 0;
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int b = kSB - 1 - 3 * lane - i;
                const uint64_t w = b >= 0 ? bin_total(b) : 0ull;
                if (w) ms += pack_mass(w, (kBin0 + (uint32_t)b) >> 2);
            }
            const u128 tot = wave_inclusive_scan(ms);
            if (lane == kWave - 1) {
                uint64_t *st = v.stash + ((size_t)row * G + part) * kStashCap;
                st[0] = (uint64_t)tot; st[1] = (uint64_t)(tot >> 64);
            }
        }
        if (tid == 0) {
            PartHdr ph;
            ph.mkey = k; ph.cov = 0u; ph.n = 0u; ph.cut = 0u;
            v.hdr[(size_t)row * G + part] = ph;
        }
        return k;
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
                put<FUSED>(&v.cum[((size_t)row * G + part) * kSB + b], nx);
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
            if (slot < (uint32_t)kStashCap) put<FUSED>(&st[slot], ((uint64_t)b << 32) | (s.gidx[i >> 2] + (i & 3u)));
        }
    }
    if (tid == 0) {
        if (FUSED) {
            uint64_t *h2 = reinterpret_cast<uint64_t *>(&v.hdr[(size_t)row * G + part]);
            a_store(&h2[0], ((uint64_t)cov << 32) | k);
            a_store(&h2[1], ((uint64_t)cut << 32) | n);
        } else {
            PartHdr ph;
            ph.mkey = k; ph.cov = cov; ph.n = n; ph.cut = cut;
            v.hdr[(size_t)row * G + part] = ph;
        }
    }
    return k;
}

template <int R, int NT, int DT, bool KEEP = false>     // NT threads, each with R groups of four tokens of the slice; DT the logits' type
__global__ void __launch_bounds__(NT, (R <= 8 ? 5 : RS_STREAM_WAVES)) stream_kernel(const Params p, const StreamView v)
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

    const bool reporter = blockIdx.x == 0 && tid == 0;
    PrevCall prev;
    prev.slow_rows = 0; prev.meta = 0;
    if (reporter) prev = report_begin(p);
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
            const uint4 l = load_once(reinterpret_cast<const uint4 *>(lg) + min(base4 + (uint32_t)(j * NT), V4 - 1));
            eb[j * 4 + 0] = l.x; eb[j * 4 + 1] = l.y; eb[j * 4 + 2] = l.z; eb[j * 4 + 3] = l.w;
        }
    } else {
        const uint2 *lh = reinterpret_cast<const uint2 *>(lrow);
        uint2 h[R];
#pragma unroll
        for (int j = 0; j < R; ++j) h[j] = load_once(lh + min(base4 + (uint32_t)(j * NT), V4 - 1));
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
    // a call that keeps everything has no rows to report on; the counting-only pass of the wide path does
    if (reporter) report_end(p, prev, !KEEP || p.report != 0u);
    slice_count_and_stash<R, NT, kRep, false, KEEP>(p, v, s, eb, lmax, row, part, base4, nv);
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
    uint32_t result;             // one-launch path: sampled token + 1 once the row is finished here
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

// A row the stashes cannot finish (a nucleus or a tie of thousands of tokens, more kept tokens than
// the list holds): the finishing workgroup does it alone, from the logits, in a few passes over the
// row -- the level-1 histogram in the row's frame (M = floor of the row's maximum is known), the
// next digits of the threshold inside the boundary bin until the bin's tokens fit a gathered list,
// the rest in LDS, then the inverse CDF by buckets of the token index, by sub-buckets, and token
// by token.  A few passes of one workgroup over one row take tens of microseconds (a row of a
// million tokens: more than a hundred): fine for the odd row, and calls whose rows mostly end here
// are routed to the cluster kernel by the caller's policy.  Same integers as every other path.
//
// KEEP_DIAG: the call keeps every live token (top_k = V, top_p = 1) and its token is picked from the
// slices' masses (keep_pick); what is left to do here is the diagnostics record, which names the
// threshold -- the smallest live token of the row -- and how many tokens tie there: one pass over
// the row, paid by callers that ask for the record (tests, mostly).  keep_live: live tokens of the row.
template <bool KEEP_DIAG = false>
__device__ __forceinline__ void finish_row_slow(const Params &p, Lds &s, LdsB &t, const uint32_t row, const float xmax, const uint64_t rand64,
                                                const uint32_t keep_live = 0u)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const float M = __builtin_floorf(xmax);
    const char *lrow = logits_row(p, row);
    const float4 *pn4 = p.penalties ? reinterpret_cast<const float4 *>(p.penalties + (int64_t)row * p.V) : nullptr;
    // bits of e of four tokens, by the definition (reference: sampling.cu:220, :553)
    auto bits_of4 = [&](const float4 l, const float4 q) -> uint4 {
        float x0, x1, x2, x3;
        if (pn4) {
            x0 = sf((sf(l.x) - q.x) * p.c); x1 = sf((sf(l.y) - q.y) * p.c); x2 = sf((sf(l.z) - q.z) * p.c); x3 = sf((sf(l.w) - q.w) * p.c);
        } else {
            x0 = sf(l.x * p.c); x1 = sf(l.y * p.c); x2 = sf(l.z * p.c); x3 = sf(l.w * p.c);
        }
        return make_uint4(e_bits_of(x0, M), e_bits_of(x1, M), e_bits_of(x2, M), e_bits_of(x3, M));
    };
    // fn(token index, bits of its e) for the tokens of groups [lo4, hi4) of the row, four loads in flight per thread
    auto row_pass = [&](uint32_t lo4, uint32_t hi4, auto fn) {
        constexpr int kAhead = 4;
        for (uint32_t base = lo4 + (uint32_t)tid; base < hi4; base += kAhead * kThreads) {
            float4 l[kAhead], q[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t i4 = min(base + (uint32_t)u * kThreads, hi4 - 1u);
                l[u] = load_logits4(lrow, i4, p.dtype);
                q[u] = pn4 ? pn4[i4] : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t i4 = base + (uint32_t)u * kThreads;
                if (i4 < hi4) {
                    const uint4 b = bits_of4(l[u], q[u]);
                    fn(i4 * 4u, b.x); fn(i4 * 4u + 1u, b.y); fn(i4 * 4u + 2u, b.z); fn(i4 * 4u + 3u, b.w);
                }
            }
        }
    };
    const uint64_t top_k = (uint64_t)p.top_k;
    if constexpr (KEEP_DIAG) {
        uint32_t mn = 0xFFFFFFFFu, cnt = 0u;
        row_pass(0u, V4, [&](uint32_t, uint32_t b) {
            if (b >= kEMinBits) {
                if (b < mn) { mn = b; cnt = 1u; }
                else if (b == mn) ++cnt;
            }
        });
        const uint32_t wm = ~wave_max_u32(~mn);
        __syncthreads();
        if (lane == 0) s.u32[wave] = wm;
        __syncthreads();
        uint32_t bm = s.u32[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) bm = min(bm, s.u32[w]);
        const uint32_t ci = wave_inclusive_scan(mn == bm ? cnt : 0u);
        __syncthreads();
        if (lane == kWave - 1) s.u32[wave] = ci;
        __syncthreads();
        if (tid == 0) {
            uint32_t n_eq = 0;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) n_eq += s.u32[w];
            const u128 D = s.D;
            tie_and_target(p, row, rand64, xmax, D, s.P, bm, keep_live - n_eq, n_eq, D - (u128)n_eq * w_of_bits(bm), 9u, true);
        }
        __syncthreads();
        return;
    }

    // level 1 (dead tokens, below 2^-40, are left out)
    __syncthreads();
    for (int b = tid; b < kNB * kRepC; b += kThreads) s.hr[b] = 0;
    __syncthreads();
    row_pass(0u, V4, [&](uint32_t, uint32_t b) {
        if (b >= kEMinBits)
            atomicAdd(reinterpret_cast<unsigned long long *>(&s.hr[(b >> 21) * kRepC + (lane & (kRepC - 1))]),
                      (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
    });
    __syncthreads();
    for (int b = tid; b < kNB; b += kThreads) {
        uint64_t w = 0;
#pragma unroll
        for (int c = 0; c < kRepC; ++c) w += s.hr[b * kRepC + c];
        s.g[b] = w;
    }
    __syncthreads();
    Found f = hist_find_level1<false>(s, top_k, p.top_p, lane, wave);
    const u128 D = s.D, P = s.P;
    const uint32_t exb = f.bin >> 2;
    uint32_t lo = f.bin << 21, span = (1u << 21) - 1u, levels = 1;
    bool one_tie = false;
    if (f.cnt_bin > (uint32_t)kCap && f.cnt_above == 0u) {
        const uint32_t emax = e_bits_of(xmax, M);
        one_tie = bin_is_one_tie(s.g[f.bin], f.bin, emax);
        if (one_tie) { lo = emax; span = 0u; }
    }
    // further digits over the whole row while the boundary bin holds more tokens than can be gathered
    while (!one_tie && f.cnt_bin > (uint32_t)kCap && levels < (uint32_t)kLevels) {
        ++levels;
        const uint32_t dsh = level_shift(levels);
        __syncthreads();
        lds_hist_zero(s, 128);
        __syncthreads();
        row_pass(0u, V4, [&](uint32_t, uint32_t b) {
            if (b - lo <= span) lds_hist_add(s, (b >> dsh) & 127u, b);
        });
        __syncthreads();
        f = hist_find128(s, s.hm, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
        lo |= f.bin << dsh;
        span = (1u << dsh) - 1u;
    }
    if (f.cnt_bin <= (uint32_t)kCap) {
        // gather the bin's tokens and resolve the remaining digits on them
        __syncthreads();
        if (tid == 0) s.ctr = 0;
        __syncthreads();
        row_pass(0u, V4, [&](uint32_t idx, uint32_t b) {
            if (b - lo <= span) {
                const uint32_t o = atomicAdd(&s.ctr, 1u);
                if (o < (uint32_t)kCap) s.cand[o] = ((uint64_t)b << 32) | idx;
            }
        });
        __syncthreads();
        const uint32_t ncand = min(s.ctr, (uint32_t)kCap);
        for (uint32_t lv = levels + 1; lv <= (uint32_t)kLevels && f.cnt_bin > 1u && span != 0u; ++lv) {
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
    const uint32_t thr = lo;
    if (tid == 0) {
        const Target tg = tie_and_target(p, row, rand64, xmax, D, P, thr, f.cnt_above, f.cnt_bin, f.mass_above, 8u, true);
        s.bc64[1] = tg.w_tie; s.bc128[0] = tg.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    u128 r = s.bc128[0];
    auto weight = [&](uint32_t b) -> uint64_t { return (b > thr) ? w_of_bits(b) : (b == thr ? w_tie : 0); };

    // inverse CDF in index order: 256 buckets of 2^sh1 tokens, 256 sub-buckets of 2^sh2, then one by one
    uint32_t sh1 = 0;
    while (((uint32_t)p.V - 1u) >> sh1 >= 256u) ++sh1;
    const uint32_t sh2 = sh1 > 8u ? sh1 - 8u : 0u;
    auto bucket_pass = [&](uint32_t lo_idx, uint32_t hi_idx, uint32_t shift) -> uint32_t {
        t.blo[tid] = 0; t.bhi[tid] = 0;
        __syncthreads();
        const uint32_t a4 = lo_idx >> 2, e4 = min(V4, (hi_idx + 3u) >> 2);
        row_pass(a4, e4, [&](uint32_t idx, uint32_t b) {
            const uint64_t w = weight(b);
            if (w && idx >= lo_idx && idx < hi_idx) {
                const uint32_t bk = (idx - lo_idx) >> shift;               // < 256: the range spans at most 256 buckets
                atomicAdd(reinterpret_cast<unsigned long long *>(&t.blo[bk]), (unsigned long long)(w & 0xFFFFFFFFull));
                atomicAdd(reinterpret_cast<unsigned long long *>(&t.bhi[bk]), (unsigned long long)(w >> 32));
            }
        });
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
        const uint32_t bk = t.bucket;
        __syncthreads();
        return bk;
    };
    const uint32_t b1 = bucket_pass(0u, (uint32_t)p.V, sh1);
    uint32_t lo_idx = b1 << sh1;
    if (sh1 > sh2) {
        const uint32_t b2 = bucket_pass(lo_idx, min((uint32_t)p.V, lo_idx + (1u << sh1)), sh2);
        lo_idx += b2 << sh2;
    }
    if (tid == 0) {
        // the last few tokens one after the other
        const uint32_t hi_idx = min((uint32_t)p.V, lo_idx + (1u << sh2));
        uint32_t pick = lo_idx;
        u128 acc = 0;
        bool found = false;
        for (uint32_t i4 = lo_idx >> 2; i4 * 4u < hi_idx && !found; ++i4) {
            const uint4 b = bits_of4(load_logits4(lrow, i4, p.dtype), pn4 ? pn4[i4] : make_float4(0.f, 0.f, 0.f, 0.f));
            auto step = [&](uint32_t idx, uint32_t bits) {
                if (found || idx < lo_idx || idx >= hi_idx) return;
                acc += weight(bits);
                if (acc >= r) { pick = idx; found = true; }
            };
            step(i4 * 4u, b.x); step(i4 * 4u + 1u, b.y); step(i4 * 4u + 2u, b.z); step(i4 * 4u + 3u, b.w);
        }
        p.out[row] = (int32_t)pick;
        if (p.diag) p.diag[row].index = (int32_t)pick;
        t.result = pick + 1u;
    }
}

// The token of a row of a call that keeps everything: the slice that begins at token lo_idx holds
// the target, r is the target's offset inside the slice.  The slice is gone through in chunks of
// 64 float4 groups (256 consecutive tokens, one KB that a wave loads in one go): chunk c belongs
// to wave c mod 4, which sums its tokens' weights (two 64-bit wave sums of the weights' halves);
// one wave scans the chunk totals for the chunk that holds the target, loads that chunk again,
// scans its 64 groups, and the lane whose group holds the target walks its four tokens.  No
// atomics, no list.  (An earlier version gave every thread 16 consecutive groups: its loads, 64
// cache lines per instruction and every line touched by 8 instructions, cost a microsecond per
// group.)  No penalties on this path.
// `kept`: weight of a token from the bit pattern of its e in the row's frame (its full weight when the
// call keeps every live token; on the wide path what the threshold and the tie weight leave of it).
template <int SLICE_LOG2, typename WF>
__device__ __forceinline__ void keep_pick(const Params &p, Lds &s, LdsB &t, const uint32_t row, const float M, const uint32_t lo_idx, const u128 r,
                                          WF kept)
{
    constexpr int N = 1 << (SLICE_LOG2 - 10);                      // chunks per wave
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const char *lrow = logits_row(p, row);
    const uint32_t g0 = lo_idx >> 2;
    auto weight = [&](float l) -> uint64_t { return kept(e_bits_of(sf(l * p.c), M)); };
    float4 l[N];
#pragma unroll
    for (int j = 0; j < N; ++j) l[j] = load_logits4(lrow, min(g0 + (uint32_t)((j * kWaves + wave) * kWave + lane), V4 - 1u), p.dtype);
#pragma unroll
    for (int j = 0; j < N; ++j) {
        uint64_t a = 0, b = 0;
        if (g0 + (uint32_t)((j * kWaves + wave) * kWave + lane) < V4) {            // past the end of the row: no weight
            const uint64_t w0 = weight(l[j].x), w1 = weight(l[j].y), w2 = weight(l[j].z), w3 = weight(l[j].w);
            a = (w0 & 0xFFFFFFFFull) + (w1 & 0xFFFFFFFFull) + (w2 & 0xFFFFFFFFull) + (w3 & 0xFFFFFFFFull);
            b = (w0 >> 32) + (w1 >> 32) + (w2 >> 32) + (w3 >> 32);
        }
        a = wave_sum(a); b = wave_sum(b);
        if (lane == 0) { t.blo[j * kWaves + wave] = a; t.bhi[j * kWaves + wave] = b; }
    }
    __syncthreads();
    if (wave == 0) {
        const u128 mine = lane < N * kWaves ? (u128)t.blo[lane] + ((u128)t.bhi[lane] << 32) : (u128)0;
        const u128 inc = wave_inclusive_scan(mine);
        const u128 exc = inc - mine;
        if (exc < r && r <= inc) { t.bucket = (uint32_t)lane; s.bc128[1] = r - exc; }
    }
    __syncthreads();
    if (wave == 0) {
        const uint32_t g = g0 + t.bucket * (uint32_t)kWave + (uint32_t)lane;
        const u128 r2 = s.bc128[1];
        uint64_t w[4] = {0ull, 0ull, 0ull, 0ull};
        if (g < V4) {
            const float4 q = load_logits4(lrow, g, p.dtype);
            w[0] = weight(q.x); w[1] = weight(q.y); w[2] = weight(q.z); w[3] = weight(q.w);
        }
        const u128 mine = (u128)w[0] + w[1] + w[2] + w[3];
        const u128 inc = wave_inclusive_scan(mine);
        u128 acc = inc - mine;
        if (acc < r2 && r2 <= inc) {
            uint32_t pick = g * 4u + 3u;
            bool found = false;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                acc += w[q];
                if (!found && acc >= r2) { pick = g * 4u + (uint32_t)q; found = true; }
            }
            p.out[row] = (int32_t)pick;
            if (p.diag) p.diag[row].index = (int32_t)pick;
            t.result = pick + 1u;
        }
    }
}

// Penalties at scale (stream_pen_kernel): the pass has already written every slice's decayed penalties and
// noted the old values that were not +0.0.  A row that has to be done the slow way needs the old values
// of all its tokens: the notes are played back, and every slice of the row is marked deferred, so that
// the fix-up kernel rewrites the whole row once its token is known.
__device__ __forceinline__ void pen_restore(const Params &p, const StreamView &v, const uint32_t row)
{
    const int tid = threadIdx.x;
    float *pen = p.penalties + (int64_t)row * p.V;
    for (uint32_t g = 0; g < v.G; ++g) {
        uint64_t *rec = v.pens + ((size_t)row * v.G + g) * kPenCap;
        const uint64_t h = rec[0];
        if (!(h & kPenDeferred))
            for (uint32_t i = (uint32_t)tid; i < (uint32_t)h; i += kThreads) {
                const uint64_t e = rec[1 + i];
                pen[(uint32_t)e] = __uint_as_float((uint32_t)(e >> 32));
            }
    }
    __syncthreads();
    if ((uint32_t)tid < v.G) v.pens[((size_t)row * v.G + tid) * kPenCap] = kPenDeferred;
    wait_vmem();
    __syncthreads();
}

// The sampled token's penalty: fma(old, decay, old == 0 ? presence : repetition) (reference:
// sampling.cu:427-437), the old value from the slice's notes (+0.0 when it is not among them).  A deferred
// slice still holds its old penalties and is rewritten whole by the fix-up kernel.
__device__ __forceinline__ void pen_patch(const Params &p, const StreamView &v, Lds &s, const uint32_t row, const uint32_t idx, const uint32_t slice_log2)
{
    const int tid = threadIdx.x;
    const uint64_t *rec = v.pens + ((size_t)row * v.G + (idx >> slice_log2)) * kPenCap;
    const uint64_t h = rec[0];
    if (h & kPenDeferred) return;
    if (tid == 0) s.bc32[6] = 0u;
    __syncthreads();
    for (uint32_t i = (uint32_t)tid; i < (uint32_t)h; i += kThreads) {
        const uint64_t e = rec[1 + i];
        if ((uint32_t)e == idx) s.bc32[6] = (uint32_t)(e >> 32);
    }
    __syncthreads();
    if (tid == 0) {
        const float old = __uint_as_float(s.bc32[6]);
        p.penalties[(int64_t)row * p.V + idx] = __builtin_fmaf(old, p.decay, old == 0.0f ? p.presence : p.repetition);
    }
}

// Finishes a row from what its slices published.  Returns true when the row is done (token written),
// false when it cannot be finished from the stashes: only on the one-launch path (FUSED = true: the
// caller is the last workgroup of the row to publish, the data was written by workgroups of this same
// launch and is read with device-scope atomic loads), where the caller then tells the row's other
// workgroups and the row's histogram is left in place for them.  With FUSED = false such a row is
// done here the slow way, from the logits.
template <int SLICE_LOG2, bool FUSED, bool KEEP = false>     // SLICE_LOG2: log2 of the tokens per slice of the view
__device__ __forceinline__ bool finish_row(const Params &p, const StreamView &v, Lds &s, LdsB &t, const uint32_t row)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const PartHdr *hdrs = v.hdr + (size_t)row * G;
    uint64_t *rowhist = FUSED ? (p.ctl_end - 1 - row)->h[0] : (p.ctl_end - 1 - row)->rowhist;

    if (tid == 0) { s.abort = 0; s.host_words = p.host_words; t.fail = 0; t.result = 0u; }
    PartHdr ph;
    ph.mkey = 0; ph.cov = 0; ph.n = 0; ph.cut = 0;
    if ((uint32_t)tid < G) {
        if (FUSED) {
            const uint64_t *h2 = reinterpret_cast<const uint64_t *>(&hdrs[tid]);
            const uint64_t w0 = a_load(&h2[0]), w1 = a_load(&h2[1]);
            ph.mkey = (uint32_t)w0; ph.cov = (uint32_t)(w0 >> 32); ph.n = (uint32_t)w1; ph.cut = (uint32_t)(w1 >> 32);
        } else ph = hdrs[tid];
    }
    const uint64_t h0 = get<FUSED>(&rowhist[tid]), h1 = get<FUSED>(&rowhist[tid + kThreads]);
    // the first lane of wave 1 draws the row's random number while wave 0 scans the histogram;
    // the state is advanced only once the row is certain to be finished here
    const bool drawer = tid == kWave && !p.inj_u;
    uint32_t *rng_st = p.rng + (size_t)row * 16;
    uint32_t rs[6] = {0u, 0u, 0u, 0u, 0u, 0u};
    if (drawer) {
#pragma unroll
        for (int i = 0; i < 6; ++i) rs[i] = rng_st[i];
    }
    if (!FUSED) { rowhist[tid] = 0; rowhist[tid + kThreads] = 0; }   // left clean for the next call
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
                    const uint64_t w = get<FUSED>(&v.shist[((size_t)row * G + g) * kSB + r]);
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
            uint4 q;
            if (FUSED) {
                const uint32_t *w = reinterpret_cast<const uint32_t *>(&eb4[i4]);
                q = make_uint4(a_load(&w[0]), a_load(&w[1]), a_load(&w[2]), a_load(&w[3]));
            } else q = eb4[i4];
            q.x = fix(q.x, d); q.y = fix(q.y, d); q.z = fix(q.z, d); q.w = fix(q.w, d);
            if (FUSED) {
                // written through: a workgroup that falls back rewrites its slice of this later
                uint32_t *w = reinterpret_cast<uint32_t *>(&eb4[i4]);
                a_store(&w[0], q.x); a_store(&w[1], q.y); a_store(&w[2], q.z); a_store(&w[3], q.w);
            } else eb4[i4] = q;
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
    // What the stashes cannot finish, this workgroup does alone from the logits.  Such rows are
    // counted, and the first of a call tells the caller's policy at once (that a call went well is
    // reported by the call after it, see report_begin).
    auto tell_policy = [&]() {
        if (tid == 0) {
            const uint32_t c = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
            if (c == 0u && p.host_words)                 // the call's first such row tells the caller's policy at once
                __hip_atomic_store(p.host_words + p.report, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    };
    auto slow = [&]() -> bool {
        if (drawer) {                                    // the row is finished here: this draw is used up
            rng_st[2] = rs[2] + 1u;
            if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
        }
        if (!FUSED && p.penalties && p.defer_pen == 2) pen_restore(p, v, row);
        finish_row_slow(p, s, t, row, xmax, p.inj_u ? 0ull : t.rand64);
        tell_policy();
        return true;
    };

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
            t.result = lo_i + 1u;
        }
        return true;
    }

    if constexpr (KEEP) {
        // Every live token is kept with its full weight (S = D).  Each slice's mass, moved into the
        // row's frame, is exact (a bin is dead in the row's frame as a whole or not at all: frames
        // differ by whole octaves); a scan over the slices finds the one that holds the target, and
        // only that slice's logits are looked at again.
        if (drawer) {
            rng_st[2] = rs[2] + 1u;
            if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
        }
        u128 mine = 0;
        if ((uint32_t)tid < G && dl < 41u) {                          // 41 octaves and more below: nothing of the slice is live
            const uint64_t *sm = v.stash + ((size_t)row * G + tid) * kStashCap;
            mine = (u128)sm[0] | ((u128)sm[1] << 64);
            if (dl) {
                // the slice's lowest 4 dl bins are dead in the row's frame; the rest is a multiple of 2^dl
                const uint64_t *sh = v.shist + ((size_t)row * G + tid) * kSB;
                u128 low = 0;
                for (uint32_t b = 0; b < 4u * dl; ++b) {
                    const uint64_t w = sh[b];
                    if (w) low += pack_mass(w, (kBin0 + b) >> 2);
                }
                mine = (mine - low) >> dl;
            }
        }
        const u128 r = p.inj_u ? ceil_mul(p.inj_u[row], D) : r_from_bits(t.rand64, D);
        u128 inc = wave_inclusive_scan(mine);
        if (lane == kWave - 1) s.q128[wave] = inc;
        __syncthreads();
        for (int w = 0; w < wave; ++w) inc += s.q128[w];
        const u128 exc = inc - mine;
        if (exc < r && r <= inc) { t.bucket = (uint32_t)tid; s.bc128[1] = r - exc; }
        __syncthreads();
        const uint32_t g = t.bucket;
        const u128 r_in = s.bc128[1];
        __syncthreads();
        if (p.diag) finish_row_slow<true>(p, s, t, row, xmax, p.inj_u ? 0ull : t.rand64, f.cnt_above + f.cnt_bin);
        keep_pick<SLICE_LOG2>(p, s, t, row, M, g << SLICE_LOG2, r_in,
                              [](uint32_t b) -> uint64_t { return b >= kEMinBits ? w_of_bits(b) : 0ull; });
        return true;
    }

    // Plan A: every stash reaches down to the row's boundary bin.  Then exactly the tokens at or
    // above that bin are taken, a prefix of each stash whose length is one cumulative count.
    uint32_t total = f.cnt_above + f.cnt_bin;
    uint32_t mtake = 0;
    bool bad = total > v.list_cap;
    if ((uint32_t)tid < G) {
        const int lb = (int)(f.bin - kBin0) + 4 * (int)dl;            // boundary bin in the slice's frame
        if (dl >= 64u) mtake = 0;                                      // the whole slice is dead in the row's frame
        else if (lb < kSB) mtake = get<FUSED>(&v.cum[((size_t)row * G + tid) * kSB + lb]);
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
    // fn(i, e in the row's frame, token) for the first n entries of the stashes' prefixes as t.take has
    // them (entry i belongs to the first slice whose inclusive prefix exceeds i): a thread takes a run of
    // consecutive entries, so that it looks up its first slice once and walks on from there, eight
    // loads in flight
    auto stashed = [&](const uint32_t n_all, auto fn) {
        constexpr int kBatch = 8;
        const uint32_t per = (n_all + kThreads - 1u) / kThreads;
        uint32_t i = (uint32_t)tid * per;
        const uint32_t iend = min(n_all, i + per);
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
                const uint64_t e = get<FUSED>(&v.stash[((size_t)row * G + g) * kStashCap + (i - gbase)]);
                fn(i, rebase_bits((uint32_t)(e >> 32), t.delta[g]), (uint32_t)e);
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
                    e[u] = get<FUSED>(&v.stash[((size_t)row * G + g) * kStashCap + (i + (uint32_t)u - gbase)]);
                    sl[u] = g;
                }
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if ((uint32_t)u < n) fn(i + (uint32_t)u, rebase_bits((uint32_t)(e[u] >> 32), t.delta[sl[u]]), (uint32_t)e[u]);
            i += n;
        }
    };
    take_prefix(mtake);
    bool subset = false;                                               // plan B in force
    bool listed = false;                                               // the list has been filled already
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
        if (!FUSED && total > min(v.list_cap, max(2048u, 3u * (uint32_t)p.top_k)) && (uint32_t)p.top_k <= v.list_cap / 2u) {
            // More stashed tokens than the list holds (a flat row cut into many slices, each of which
            // stashed several times its share of top_k), or several times top_k of them (going through
            // a list of thousands a dozen times costs more than these two passes: 128 flat rows of
            // 100256 with top_k 1000, 60 against 70 us).  The kept set is at most top_k tokens, so only
            // the stashed tokens down to some value T at or above which there are at least top_k of
            // them are needed: T from a count of the stashed tokens in steps of 1/512 octave below the
            // row's largest (one pass over the stashes, which sit in the L2), the tokens at or above T
            // into the list by a second pass.  T is at or above cutrow, so the list is complete above T.
            const uint32_t topkey = e_bits_of(xmax, M) >> 14;
            uint32_t *cnt = reinterpret_cast<uint32_t *>(t.blo);                // 512 counters
            cnt[tid] = 0u; cnt[tid + kThreads] = 0u;
            if (tid == 0) { s.ctr = 0u; s.bc32[4] = 0xFFFFFFFFu; s.bc32[5] = 0u; }
            __syncthreads();
            stashed(total, [&](uint32_t, uint32_t b, uint32_t) {
                if (b >= cutrow) atomicAdd(&cnt[min(511u, topkey - (b >> 14))], 1u);
            });
            __syncthreads();
            if (wave == 0) {
                uint32_t c8 = 0;
#pragma unroll
                for (int q = 0; q < 8; ++q) c8 += cnt[lane * 8 + q];
                const uint32_t inc = wave_inclusive_scan(c8);
                uint32_t run = inc - c8;
                if (run < (uint32_t)p.top_k && (uint32_t)p.top_k <= inc) {
                    bool done = false;
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        run += cnt[lane * 8 + q];
                        if (!done && run >= (uint32_t)p.top_k) { s.bc32[4] = (uint32_t)(lane * 8 + q); s.bc32[5] = run; done = true; }
                    }
                }
            }
            __syncthreads();
            const uint32_t step = s.bc32[4], nge = s.bc32[5];
            if (step >= 511u || nge > v.list_cap) return slow();              // fewer than top_k at or above cutrow, or one value thousands of times
            cutrow = max(cutrow, (topkey - step) << 14);
            stashed(total, [&](uint32_t, uint32_t b, uint32_t idx) {
                if (b >= cutrow) {
                    const uint32_t o = atomicAdd(&s.ctr, 1u);
                    if (o < v.list_cap) t.list[o] = ((uint64_t)b << 32) | idx;
                }
            });
            __syncthreads();
            total = nge;
            subset = true; listed = true;
            // Two more passes over the stashes make this finish slower than the general kernel's whole
            // call while the call is of moderate size (measured: 64 flat rows of 131072 with top_k 1000,
            // 51 against 38 us; 128 rows of 262144, 77 against 117): such a call says so to the caller's
            // policy, as it did when these rows still went the slow way.
            // (p.tell_lists: calls of fewer than 2^24 tokens, and calls whose rows the row kernel would take)
            if (p.tell_lists) tell_policy();
        } else {
        if (total > v.list_cap || total == 0u) {
            // not resolvable from the stashes
            if (FUSED) return false;
            return slow();
        }
        subset = true;
        }
    }

    // A nucleus of thousands of tokens is finished here all the same, but one workgroup going through
    // such a list a dozen times takes longer than the general kernel needs for the whole call (measured:
    // 128 rows of 50304, about 4000 tokens each, 54 against 36 us; the two meet at about 2400 tokens
    // there and, the general kernel's time growing with the row, at about 4700 for rows of 100256): a
    // call that is only an attempt (no top_k bounds the kept set) says so to the caller's policy, and so
    // does a call of moderate size with a bounding top_k (a lone flat row of 32768 tokens with top_k 1000:
    // 26.7 us here against 17.5 on the general kernel).  Small calls in rows of up to 100256 tokens meet the
    // general kernel earlier: a list of a thousand tokens takes one to sixteen such rows 21-27 us here
    // against 18-21 there (lists of a few hundred: 12-14 us here).
    const bool small_call = (uint64_t)p.B * (uint64_t)p.V < (1ull << 20) && p.V < 131072;
    const uint32_t long_list = small_call ? 768u : max(2048u, (uint32_t)p.V / 20u);
    if (!FUSED && (p.attempt || p.tell_lists) && total > long_list) tell_policy();

    // gather the tokens, re-based to the row's frame
    if (!listed)
        stashed(total, [&](uint32_t i, uint32_t b, uint32_t idx) {
            if (b < cutrow) b = 0;                                     // plan B: below the complete part; 0 matches nothing
            t.list[i] = ((uint64_t)b << 32) | idx;
        });
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
            if (FUSED) return false;
            return slow();
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
            t.result = (uint32_t)me + 1u;
        }
    }
    return true;
}

template <int SLICE_LOG2, bool KEEP = false>
__global__ void __launch_bounds__(kThreads) finish_kernel(const Params p, const StreamView v)
{
    __shared__ Lds s;
    __shared__ LdsB t;
    extern __shared__ __align__(16) unsigned char finish_dyn[];
    t.list = reinterpret_cast<uint64_t *>(finish_dyn);       // every thread writes the same value (KEEP: no list, not used)
    finish_row<SLICE_LOG2, false, KEEP>(p, v, s, t, blockIdx.x);
    if (!KEEP && p.penalties && p.defer_pen == 2) {
        __syncthreads();
        pen_patch(p, v, s, blockIdx.x, t.result - 1u, SLICE_LOG2);
    }
}



// The streaming pass for calls with penalties too large for the one-launch path: logits and penalties
// are read once, x = sf((sf(l) - pen) * c) as in the cluster kernel, everything after that is the
// streaming pass.  The sampled token is not known yet, but every OTHER token's new penalty is
// fma(pen, decay, 0), so the pass writes those from its registers -- 12 bytes per token in all, as the
// reference's single kernel moves (sampling.cu:211,220,427-437) -- and the finishing workgroup patches the
// one sampled token.  That needs the sampled token's old value, and a row the finishing workgroup has to do
// the slow way needs the old values of all its tokens; penalties are non-zero only where tokens have been
// generated, so each slice notes the old values whose bit pattern is not +0.0 (up to kPenCap - 1 of them; a
// slice with more leaves its penalties untouched and says so, and penalty_fix_kernel rewrites such slices
// once the tokens are known).  Groups of four that are all +0.0 stay +0.0 under a finite decay and are
// not written at all.
template <int R>
__global__ void __launch_bounds__(kThreads, 2) stream_pen_kernel(const Params p, const StreamView v)
{
    constexpr int kRep = stream_copies<R>();
    __shared__ LdsA<kRep> s;
    __shared__ uint64_t noted[kWaves][kPenWave];
    __shared__ uint32_t nnote[kWaves];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const bool reporter = blockIdx.x == 0 && threadIdx.x == 0;
    PrevCall prev;
    prev.slow_rows = 0; prev.meta = 0;
    if (reporter) prev = report_begin(p);
    Slice<R, true> sl;
    slice_setup(p, sl, row, part, G);
    const float lmax = slice_load(p, sl);
    if (reporter) report_end(p, prev, true);
    if (p.defer_pen == 2) {
        // the penalties whose bit pattern is not +0.0, side by side into this wave's notes
        uint32_t fill = 0;                               // wave-uniform: every lane takes part in every vote
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t b4[4] = {__float_as_uint(sl.pen[j].x), __float_as_uint(sl.pen[j].y), __float_as_uint(sl.pen[j].z), __float_as_uint(sl.pen[j].w)};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bool nz = j < sl.nv && b4[q] != 0u;
                const uint64_t vote = __ballot(nz);
                if (nz) {
                    const uint32_t pos = fill + __builtin_amdgcn_mbcnt_hi((uint32_t)(vote >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)vote, 0u));
                    if (pos < (uint32_t)kPenWave) noted[wave][pos] = ((uint64_t)b4[q] << 32) | ((sl.base4 + (uint32_t)j * kThreads) * 4u + (uint32_t)q);
                }
                fill += (uint32_t)__popcll(vote);
            }
        }
        if (lane == 0) nnote[wave] = fill;
        __syncthreads();
        uint32_t total = 0, before = 0;
        bool fits = true;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t n = nnote[w];
            if (w < wave) before += n;
            total += n;
            fits = fits && n <= (uint32_t)kPenWave;
        }
        fits = fits && total < (uint32_t)kPenCap;
        uint64_t *rec = v.pens + ((size_t)row * G + part) * kPenCap;
        if (fits) {
            for (uint32_t i = (uint32_t)lane; i < fill; i += kWave) rec[1 + before + i] = noted[wave][i];
            if (tid == 0) rec[0] = total;
#pragma unroll
            for (int j = 0; j < R; ++j) {
                float4 q = sl.pen[j];
                if (j < sl.nv && (__float_as_uint(q.x) | __float_as_uint(q.y) | __float_as_uint(q.z) | __float_as_uint(q.w)) != 0u) {
                    q.x = __builtin_fmaf(q.x, p.decay, 0.0f); q.y = __builtin_fmaf(q.y, p.decay, 0.0f);
                    q.z = __builtin_fmaf(q.z, p.decay, 0.0f); q.w = __builtin_fmaf(q.w, p.decay, 0.0f);
                    sl.pn4[sl.base4 + (uint32_t)j * kThreads] = q;
                }
            }
        } else if (tid == 0) rec[0] = kPenDeferred;
    }
    slice_count_and_stash<R, kThreads, kRep, false>(p, v, s, sl.eb, lmax, row, part, sl.base4, sl.nv);
}

// pen <- fma(pen, decay, onehot * (pen == 0 ? presence : repetition)), the switch on the value before
// the decay (reference: sampling.cu:427-437), from the sampled token in p.out, for the slices that still
// hold their old penalties: all of them when the streaming pass left the penalties alone (defer_pen 1),
// else those marked deferred -- by the pass (too many non-zero penalties to note) or by the finishing
// workgroup of a row done the slow way (which played the notes back).  One workgroup per slice; the others
// leave after one load.
template <int R>
__global__ void __launch_bounds__(kThreads) penalty_fix_kernel(const Params p, const StreamView v)
{
    const uint32_t G = v.G;
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    if (p.defer_pen == 2 && !(v.pens[((size_t)row * G + part) * kPenCap] & kPenDeferred)) return;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t idx = (uint32_t)p.out[row];
    float4 *pn4 = reinterpret_cast<float4 *>(p.penalties + (int64_t)row * p.V);
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + threadIdx.x;
    float4 q[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint32_t i4 = base4 + (uint32_t)j * kThreads;
        if (i4 < V4) q[j] = pn4[i4];
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint32_t i4 = base4 + (uint32_t)j * kThreads;
        if (i4 < V4) {
            float4 w = q[j];
            const uint32_t e0 = i4 * 4;
            w.x = __builtin_fmaf(w.x, p.decay, (e0 + 0 != idx) ? 0.0f : (w.x == 0.0f ? p.presence : p.repetition));
            w.y = __builtin_fmaf(w.y, p.decay, (e0 + 1 != idx) ? 0.0f : (w.y == 0.0f ? p.presence : p.repetition));
            w.z = __builtin_fmaf(w.z, p.decay, (e0 + 2 != idx) ? 0.0f : (w.z == 0.0f ? p.presence : p.repetition));
            w.w = __builtin_fmaf(w.w, p.decay, (e0 + 3 != idx) ? 0.0f : (w.w == 0.0f ? p.presence : p.repetition));
            pn4[i4] = w;
        }
    }
}

// ------------------------------------------------------------ one-launch path --
// The streaming pass and the finish in ONE launch, for calls small enough that a second and a third
// launch (and the cold start of the finishing workgroup) cost as much as the work itself, and for
// calls with penalties, whose every workgroup needs the sampled token to rewrite its penalties from
// the registers.  A row is worked by G workgroups (logical ids follow the order in which workgroups
// start once the launch is larger than the GPU holds at once).  Each reads its slice once, publishes
// the slice's record exactly as the streaming pass does -- with device-scope atomic stores -- and
// counts itself in (release).  The workgroup that arrives last finishes the row from the records
// (acquire; finish_row) and posts a verdict: the sampled token, or "fall back".  The others wait for
// the verdict -- that is the only wait, and it is for a workgroup that is already running.  On "fall
// back" (a nucleus or a tie too large for the stashes) all G workgroups go on with the cluster path's
// rounds from the tokens they still hold in registers: the row's level-1 histogram is already
// complete in memory, so they start at the boundary search.  With penalties every workgroup then
// rewrites its slice of them.  The last workgroup to leave cleans the row's record.
template <int R, bool PEN>
struct FusedLds {
    union {
        LdsA<stream_copies<R>()> a;
        struct { Lds s; LdsB t; } f;
    };
};

template <int R, bool PEN>
__device__ __forceinline__ bool fused_fallback(const Params &p, const StreamView &v, Lds &s, Slice<R, PEN> &sl, uint32_t slice_key)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = sl.G, row = sl.row, part = sl.part;
    RowCtl *rc = sl.rc;
    draw_rand(p, s, row);
    // the slices' maxima, the row's level-1 histogram (complete: every workgroup has arrived) and
    // this slice's own bins, all as they were published
    uint32_t mk = 0;
    if ((uint32_t)tid < G) mk = (uint32_t)a_load(reinterpret_cast<const uint64_t *>(&v.hdr[(size_t)row * G + tid]));
    const uint64_t g0 = a_load(&rc->h[0][tid]), g1 = a_load(&rc->h[0][tid + kThreads]);
    uint64_t mine = 0;
    if (tid < kSB) mine = a_load(&v.shist[((size_t)row * G + part) * kSB + tid]);
    uint32_t kmax, kmin;
    {
        const uint32_t a = wave_max_u32(mk), b = wave_max_u32((uint32_t)tid < G ? ~mk : 0u);
        __syncthreads();
        if (lane == 0) { s.u32[wave] = a; s.u32[kWaves + wave] = b; }
        __syncthreads();
        kmax = s.u32[0]; kmin = s.u32[kWaves];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { kmax = max(kmax, s.u32[w]); kmin = max(kmin, s.u32[kWaves + w]); }
        kmin = ~kmin;
    }
    const float M = __builtin_floorf(fkey_inv(kmax)), Mloc = __builtin_floorf(fkey_inv(slice_key));
    const float dd = M - Mloc;
    const uint32_t delta = dd >= 64.0f ? 64u : (uint32_t)dd;
    // the registers hold e unclamped in the slice's frame: into the row's frame, dead tokens at 2^-41
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int k = 0; k < 4; ++k) sl.eb[j * 4 + k] = rebase_bits(min(sl.eb[j * 4 + k], 0x3FFFFFFFu), delta);
    sl.kmax_row = kmax;
    sl.h_used = 1u;                                      // the row's level-1 histogram is to be cleared
    sl.mx_posted = false;
    auto clear_used = [&]() {
        for (uint32_t i = 0; i <= (uint32_t)kLevels; ++i)
            if (sl.h_used >> i & 1u) zero_slice(rc->h[i], (i == 0u || i == (uint32_t)kLevels) ? (uint32_t)kNB : 128u, part, G);
        sl.h_used = 0u;
    };
    if (M - __builtin_floorf(fkey_inv(kmin)) < 88.0f) {
        // positions by absolute octave are unambiguous: both histograms into the row's frame
        const uint32_t m4 = (uint32_t)(int)(M - 128.0f * __builtin_floorf(M * 0.0078125f)) * 4u;
        const uint32_t r0 = ((uint32_t)tid + 160u - m4) & 511u, r1 = ((uint32_t)tid + kThreads + 160u - m4) & 511u;
        for (int b = tid; b < kNB; b += kThreads) { s.g[b] = 0; s.hm[b] = 0; }
        __syncthreads();
        if (r0 < 164u) s.g[kBin0 + r0] = g0;
        if (r1 < 164u) s.g[kBin0 + r1] = g1;
        if (tid < kSB && (uint32_t)tid >= 4u * delta && delta < 64u) s.hm[kBin0 + (uint32_t)tid - 4u * delta] = mine;
        __syncthreads();
    } else {
        // slices too far apart for shared positions: level 1 again, in the row's frame, through the
        // spare histogram (every token is counted, dead ones too, so that the counts add up)
        __syncthreads();
        lds_hist_zero(s, kNB);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < sl.nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t b = opaque(sl.eb[j * 4 + k]);
                    lds_hist_add(s, b >> 21, b);
                }
            }
        if (!hist_combine(s, p.hdr, G, rc->h[kLevels], kNB, (uint32_t)p.V, lane, wave)) return false;
        clear_used();                                    // every workgroup has read the first histogram before it published this one
        sl.h_used = 1u << kLevels;
    }
    return slice_finish(p, s, sl);
}

template <int R, bool PEN>
__global__ void __launch_bounds__(kThreads, 2) fused_kernel(const Params p, const StreamView v)
{
    constexpr int kRep = stream_copies<R>();
    constexpr int kSliceLog2 = R == 16 ? 14 : R == 8 ? 13 : 12;
    static_assert(R == 4 || R == 8 || R == 16, "slices of 4096, 8192 or 16384 tokens");
    __shared__ FusedLds<R, PEN> u;
    const int tid = threadIdx.x;
    const uint32_t G = v.G;
    // logical id: the hardware's while the device holds the whole launch at once (every call routed here
    // by itself does), else a ticket, so that a row's workgroups are always the next ones to start
    uint32_t id = blockIdx.x;
    constexpr uint32_t kResident = 256u * (R == 16 && PEN ? 2u : 3u);     // workgroups of this kernel the device holds at once
    if (gridDim.x > kResident) {
        if (tid == 0) {
            u.a.u32[8] = take_ticket(p.hdr);
        }
        __syncthreads();
        id = u.a.u32[8];
    }
    const uint32_t row = id / G, part = id - row * G;
    Slice<R, PEN> sl;
    slice_setup(p, sl, row, part, G);
    RowCtl *rc = sl.rc;
    const float lmax = slice_load(p, sl);
    const uint32_t key = slice_count_and_stash<R, kThreads, kRep, true>(p, v, u.a, sl.eb, lmax, row, part, sl.base4, sl.nv);

    // Count this slice in.  Everything it published went out as device-scope atomic stores (written
    // through to the level all XCDs share) and has been acknowledged before the count is raised; the
    // finishing workgroup reads with device-scope atomic loads.  No cache write-back or invalidation
    // is needed for that, and none is asked for: a release here would write back the whole L2.
#ifndef RS_FUSED_RELAXED
#define RS_FUSED_RELAXED 1
#endif
    wait_vmem();
    __syncthreads();
    if (tid == 0)
        u.a.u32[9] = RS_FUSED_RELAXED ? __hip_atomic_fetch_add(&rc->arrived, 1u, __ATOMIC_RELAXED, RS_AGENT)
                                      : __hip_atomic_fetch_add(&rc->arrived, 1u, __ATOMIC_ACQ_REL, RS_AGENT);
    __syncthreads();
    const bool last = u.a.u32[9] == G - 1u;
    __syncthreads();                                     // the LDS of the streaming pass is given up here
    Lds &s = u.f.s;
    LdsB &t = u.f.t;
    if (tid == 0) { s.abort = 0; s.host_words = p.host_words; s.who = row << 16 | part; s.seen = 0; s.want = 0; }
    uint32_t verdict = 0;
    if (last) {
        // the token list: the cluster rounds' histogram copies, which are not in use while a row is
        // finished from the stashes (no dynamic LDS in this kernel: see rs_sample_ex)
        static_assert(sizeof(s.hr) == 2048 * sizeof(uint64_t), "room for a list of 2048 tokens");
        t.list = s.hr;
        const bool done = finish_row<kSliceLog2, true>(p, v, s, t, row);
        __syncthreads();
        verdict = done && t.result != 0u ? t.result : kVerdictFallback;
        if (tid == 0) a_store(&rc->verdict, verdict);
    } else {
        __syncthreads();
        if (tid == 0) {
            const uint64_t t0 = wall_clock64();
            uint32_t spins = 0, w;
            while ((w = a_load(&rc->verdict)) == 0u) {
                __builtin_amdgcn_s_sleep(2);
                if ((++spins & 255u) == 0 && (uint64_t)wall_clock64() - t0 > spin_limit(p.hdr)) { give_up(s, p.hdr, 6u); break; }
            }
            s.bc32[7] = w;
        }
        __syncthreads();
        if (s.abort) return;
        verdict = s.bc32[7];
    }
    if (verdict == kVerdictFallback) {
        fused_fallback<R, PEN>(p, v, s, sl, key);       // ends with the cluster path's own leaving protocol
        return;
    }
    const uint32_t idx = verdict - 1u;
    if (PEN) {
        // penalties: decay and one-hot add, from registers (reference: sampling.cu:427-437)
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j < sl.nv) {
                const uint32_t i4 = sl.base4 + (uint32_t)j * kThreads;
                float4 q = sl.pen[j];
                const uint32_t e0 = i4 * 4;
                q.x = __builtin_fmaf(q.x, p.decay, (e0 + 0 != idx) ? 0.0f : (q.x == 0.0f ? p.presence : p.repetition));
                q.y = __builtin_fmaf(q.y, p.decay, (e0 + 1 != idx) ? 0.0f : (q.y == 0.0f ? p.presence : p.repetition));
                q.z = __builtin_fmaf(q.z, p.decay, (e0 + 2 != idx) ? 0.0f : (q.z == 0.0f ? p.presence : p.repetition));
                q.w = __builtin_fmaf(q.w, p.decay, (e0 + 3 != idx) ? 0.0f : (q.w == 0.0f ? p.presence : p.repetition));
                sl.pn4[i4] = q;
            }
        }
    }
    // leave: the last workgroup out of the row puts its record back to zero
    __syncthreads();
    if (tid == 0) s.bc32[0] = __hip_atomic_fetch_add(&rc->done, 1u, __ATOMIC_RELAXED, RS_AGENT);
    __syncthreads();
    if (s.bc32[0] == G - 1u) {
        a_store(&rc->h[0][tid], (uint64_t)0); a_store(&rc->h[0][tid + kThreads], (uint64_t)0);
        if (tid == 0) { a_store(&rc->done, 0u); a_store(&rc->arrived, 0u); a_store(&rc->verdict, 0u); }
    }
}

}  // namespace rs
