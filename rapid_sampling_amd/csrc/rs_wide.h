// The wide path: kept sets of thousands of tokens (top_k in the thousands, flat distributions under
// top_p) without a wait and without a list of thousands of tokens in one workgroup.
//
//   stream_kernel<.., KEEP>   the counting-only pass of the streaming path: the row's level-1
//                             histogram, each slice's own bins and maximum.
//   wide_kernel               one workgroup per slice, over the logits again (for calls of up to a
//                             few hundred MB they come from the L2 / Infinity Cache).  Every workgroup
//                             first works out, from what the first pass left, the row's frame and
//                             the boundary bin of level 1 -- the same few thousand integer operations
//                             in every workgroup of the row, while its loads are in flight.  Then it
//                             counts its tokens of that bin by their next 7 bits (added to the row's
//                             level-2 histogram, and kept as running sums under the slice's name),
//                             and sets aside the tokens of the sub-bins around the one in which it
//                             EXPECTS the row's threshold: the slice scales its own counts and masses
//                             to the row's size.  The guess decides only what is set aside; the
//                             window it covers is on record.
//   wide_finish_kernel        one workgroup per row: boundary sub-bin from the row's level-2
//                             histogram (exact), the tokens of that sub-bin from every slice's
//                             window -- a few hundred at most for a smooth distribution, whatever the
//                             size of the kept set --, the remaining 14 bits of the threshold on them,
//                             tie weight and target, the slice that holds the target from per-slice
//                             kept weights (mass above the bin from the first pass's bins, mass above
//                             the sub-bin from the running sums, the listed tokens above the
//                             threshold), and one more look at that slice's logits for the token.
//                             A row whose threshold sub-bin some slice did not cover (slices that are
//                             no fair samples of their row), or whose sub-bin holds more tokens than
//                             the list, is done the slow way and reported to the caller's policy.
// Same integers as every other path.
#pragma once

#include "rs_stream.h"

namespace rs {

constexpr int      kWideHead  = 132;                     // words at the head of a slice's stash region: kept mass above the bin (2), running sums (129)
constexpr int      kWideCap   = kStashCap - kWideHead;   // tokens a slice can set aside
constexpr int      kWideRep   = 4;                       // copies of each sub-bin while it is counted
constexpr uint32_t kWideValid = 1u << 16;                // PartHdr::cov of a slice the second pass has been over: window lo | hi << 8 | this

// What the plan kernel leaves for a row (in the first words of RowCtl::A, which the wide path does not
// use otherwise; the finishing workgroup puts them back to zero).
struct WidePlan {
    uint32_t kmax;            // fkey of the row's largest x
    uint32_t b1;              // boundary bin of level 1
    uint32_t cnt_above, cnt_bin;
    uint32_t skip;            // 1: the row is one tie of all its tokens, finished without a second pass
    float    x_lo, x_hi;      // a token lies in the boundary bin exactly when x_lo <= x < x_hi (e is monotone in x)
    float    need_mf;         // (P - mass above the bin) in units of the bin's exponent, rounded: for the slices' estimates only
    uint64_t mass_above[2], P[2], D[2];
};
static_assert(sizeof(WidePlan) <= sizeof(uint64_t) * 2 * kMaxParts, "fits RowCtl::A");

struct LdsP {                         // plan kernel
    u128     D, P;
    Found    found;
    uint64_t g[kNB];                  // the row's level-1 histogram in the row's frame
    uint32_t delta[kMaxParts], m4[kMaxParts];
    uint32_t u32[16];
};

// NW waves, each with a queue of Q entries: a quarter of the tokens a wave holds of the longest slice it is used for
template <int NW, int Q>
struct LdsW {                         // second pass
    uint32_t qx[NW][Q];               // per wave: its tokens of the boundary bin, x (then the bits of e)
    uint16_t qi[NW][Q];               // and their place in the slice: (group j * 4 + element) * threads + thread
    uint64_t sub[128 * kWideRep];     // this slice's tokens of the boundary bin by their next 7 bits
    uint64_t cp[130];                 // cp[j]: packed (count, fraction sum) of the slice's tokens in sub-bins >= j; cp[128] = 0
    uint64_t stage[kWideCap];         // the tokens set aside, ordered by sub-bin, before they are written out
    uint32_t off[128];                // where the next token of sub-bin j goes
    uint32_t win_lo, win_hi, n, over;
};

// Brings a row's level-1 histogram, as the first pass left it (positions by absolute octave mod 128),
// into the row's frame: bin r sits at position 4 (M mod 128) + r - 160.  h0, h1: positions tid and
// tid + 256.  With `mixed` (slices whose maxima lie 88 octaves or more apart may have put different
// octaves into one position) what every slice 41 octaves or more below the row's frame added is taken
// out again bin by bin: all its tokens are dead in the row's frame.  delta[], m4[]: per slice, octaves
// below the row's frame (capped at 64) and 4 (M_slice mod 128).
template <typename L>
__device__ __forceinline__ void level1_to_row_frame(L &s, const StreamView &v, const uint32_t row, const float M, const bool mixed,
                                                    const uint64_t h0, const uint64_t h1, const uint32_t *delta, const uint32_t *m4s)
{
    const int tid = threadIdx.x;
    const uint32_t G = v.G;
    const float mm = M - 128.0f * __builtin_floorf(M * 0.0078125f);
    const uint32_t m4 = (uint32_t)(int)mm * 4u;
    const uint32_t r0 = ((uint32_t)tid + 160u - m4) & 511u, r1 = ((uint32_t)tid + kThreads + 160u - m4) & 511u;
    if (r0 < (uint32_t)kSB) s.g[kBin0 + r0] = h0;
    if (r1 < (uint32_t)kSB) s.g[kBin0 + r1] = h1;
    __syncthreads();
    if (mixed) {
        for (uint32_t i = (uint32_t)tid; i < G * (uint32_t)kSB; i += kThreads) {
            const uint32_t g = i / (uint32_t)kSB, r = i - g * (uint32_t)kSB;
            if (delta[g] >= 41u) {
                const uint64_t w = v.shist[((size_t)row * G + g) * kSB + r];
                if (w) {
                    const uint32_t rr = (m4s[g] + r - m4) & 511u;
                    if (rr < (uint32_t)kSB)
                        atomicAdd(reinterpret_cast<unsigned long long *>(&s.g[kBin0 + rr]), 0ull - (unsigned long long)w);
                }
            }
        }
        __syncthreads();
    }
}

// One workgroup per row, between the two passes: the row's frame and its level-1 boundary (the bin in
// which the kept set becomes sufficient, what lies above it, the row total D and P = ceil(top_p D))
// from the first pass's records, left where every workgroup of the second pass reads them.
__global__ void __launch_bounds__(kThreads) wide_plan_kernel(const Params p, const StreamView v)
{
    __shared__ LdsP s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G, row = blockIdx.x;
    RowCtl *rc = p.ctl_end - 1 - row;
    uint32_t mk = 0;
    if ((uint32_t)tid < G) mk = v.hdr[(size_t)row * G + tid].mkey;
    const uint64_t h0 = rc->rowhist[tid], h1 = rc->rowhist[tid + kThreads];
    rc->rowhist[tid] = 0; rc->rowhist[tid + kThreads] = 0;      // left clean for the next call
    uint32_t kmax, kmin;
    {
        const uint32_t a = wave_max_u32(mk), b = wave_max_u32((uint32_t)tid < G ? ~mk : 0u);
        if (lane == 0) { s.u32[wave] = a; s.u32[kWaves + wave] = b; }
        __syncthreads();
        kmax = s.u32[0]; kmin = s.u32[kWaves];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { kmax = max(kmax, s.u32[w]); kmin = max(kmin, s.u32[kWaves + w]); }
        kmin = ~kmin;
    }
    const float xmax = fkey_inv(kmax);
    const float M = __builtin_floorf(xmax);
    const bool mixed = !(M - __builtin_floorf(fkey_inv(kmin)) < 88.0f);
    if ((uint32_t)tid < G) {
        const float Mg = __builtin_floorf(fkey_inv(mk));
        const float d = M - Mg;
        s.delta[tid] = d >= 64.0f ? 64u : (uint32_t)d;
        s.m4[tid] = (uint32_t)(int)(Mg - 128.0f * __builtin_floorf(Mg * 0.0078125f)) * 4u;
    }
    __syncthreads();
    level1_to_row_frame(s, v, row, M, mixed, h0, h1, s.delta, s.m4);
    const Found f = hist_find_level1<false, false, LdsP>(s, (uint64_t)p.top_k, p.top_p, lane, wave);
    if (tid == 0) {
        WidePlan *pl = reinterpret_cast<WidePlan *>(rc->A);
        pl->kmax = kmax; pl->b1 = f.bin; pl->cnt_above = f.cnt_above; pl->cnt_bin = f.cnt_bin;
        // a row that is one tie of all its tokens is finished without a second pass over it
        pl->skip = f.cnt_bin == (uint32_t)p.V && bin_is_one_tie(s.g[f.bin], f.bin, e_bits_of(xmax, M)) ? 1u : 0u;
        pl->mass_above[0] = (uint64_t)f.mass_above; pl->mass_above[1] = (uint64_t)(f.mass_above >> 64);
        pl->P[0] = (uint64_t)s.P; pl->P[1] = (uint64_t)(s.P >> 64);
        pl->D[0] = (uint64_t)s.D; pl->D[1] = (uint64_t)(s.D >> 64);
        const u128 units = (s.P - f.mass_above) >> ((f.bin >> 2) - 87u);
        pl->need_mf = (float)(uint64_t)(units >> 64) * 18446744073709551616.0f + (float)(uint64_t)units;
    }
    // The bin in terms of x: e is a monotone function of x (every Horner step rounds a monotone exact
    // value, the scaling is exact, octaves join below 2), so the tokens of bin b1 are those with
    // x_lo <= x < x_hi, x_lo the smallest x whose e reaches the bin and x_hi the smallest whose e reaches
    // the next one (+inf when the row's largest token does not).  Wave 0 looks for the first, wave 1 for
    // the second, over the order-preserving keys of x, 64 probes a round: six rounds for 32 bits.
    if (wave < 2) {
        const uint32_t target = (f.bin + (uint32_t)wave) << 21;
        float bound = __builtin_inff();
        if (e_bits_of(xmax, M) >= target) {
            uint64_t lo = (uint64_t)fkey(-3.402823466e+38f) - 1u, hi = kmax;      // the answer lies in (lo, hi]; e(hi) reaches the target
            while (hi - lo > 1u) {
                const uint64_t step = (hi - lo + 63u) >> 6;
                const uint64_t c = min(lo + (uint64_t)(lane + 1) * step, hi);        // lane 63 probes hi itself
                const uint64_t vote = __ballot(e_bits_of(fkey_inv((uint32_t)c), M) >= target);
                const uint64_t first = (uint64_t)(__ffsll((unsigned long long)vote) - 1);
                hi = min(lo + (first + 1u) * step, hi);
                lo = lo + first * step;
            }
            bound = fkey_inv((uint32_t)hi);
        }
        if (lane == 0) {
            WidePlan *pl = reinterpret_cast<WidePlan *>(rc->A);
            if (wave == 0) pl->x_lo = bound; else pl->x_hi = bound;
        }
    }
}

template <int R, int NT, int DT>      // NT threads, each with R groups of four tokens of the slice
__global__ void __launch_bounds__(NT) wide_kernel(const Params p, const StreamView v)
{
    constexpr int kQ = 64 * R;                           // a quarter of a wave's 4 R 64 tokens
    constexpr int kThreads = NT;                         // (shadows the namespace's: this kernel's workgroup size)
    __shared__ LdsW<NT / kWave, kQ> s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + (uint32_t)tid;
    const int nv = base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - base4 + kThreads - 1) / kThreads);
    const char *lrow = logits_row(p, row);
    RowCtl *rc = p.ctl_end - 1 - row;
    uint64_t *st = v.stash + ((size_t)row * G + part) * kStashCap;

    uint32_t eb[R * 4];
    if constexpr (DT == RS_DTYPE_F32) {
        const uint4 *lg = reinterpret_cast<const uint4 *>(lrow);
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint4 l = load_once(lg + min(base4 + (uint32_t)(j * kThreads), V4 - 1));
            eb[j * 4 + 0] = l.x; eb[j * 4 + 1] = l.y; eb[j * 4 + 2] = l.z; eb[j * 4 + 3] = l.w;
        }
    } else {
        const uint2 *lh = reinterpret_cast<const uint2 *>(lrow);
        uint2 h[R];
#pragma unroll
        for (int j = 0; j < R; ++j) h[j] = load_once(lh + min(base4 + (uint32_t)(j * kThreads), V4 - 1));
#pragma unroll
        for (int j = 0; j < R; ++j) widen4(h[j], DT, &eb[j * 4]);
    }
    // the slice's own bins from the first pass (wave 1 turns them into the slice's kept mass at the end)
    uint64_t own_bins[3] = {0ull, 0ull, 0ull};
    if (wave == 1) {
        const uint64_t *sh = v.shist + ((size_t)row * G + part) * kSB;
#pragma unroll
        for (int i = 0; i < 3; ++i) { const int t = kSB - 1 - 3 * lane - i; if (t >= 0) own_bins[i] = sh[t]; }
    }
    const uint32_t own_key = v.hdr[(size_t)row * G + part].mkey;
    for (int i = tid; i < 128 * kWideRep; i += kThreads) s.sub[i] = 0;
    if (tid == 0) s.over = 0u;
    const WidePlan *pl = reinterpret_cast<const WidePlan *>(rc->A);
    const uint32_t b1 = pl->b1, exb = b1 >> 2;
    const bool skip = pl->skip != 0u;
    const float M = __builtin_floorf(fkey_inv(pl->kmax));
    const float x_lo = pl->x_lo, x_hi = pl->x_hi;
    __syncthreads();

    // x = l * c unless a NaN or an infinity shows up (see stream_kernel)
    constexpr int kSpecial = 0x207;
    float probe = 0.0f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const float x0 = __uint_as_float(eb[j * 4]) * p.c, x1 = __uint_as_float(eb[j * 4 + 1]) * p.c;
        const float x2 = __uint_as_float(eb[j * 4 + 2]) * p.c, x3 = __uint_as_float(eb[j * 4 + 3]) * p.c;
        probe = __builtin_fmaf(x0, x1, probe);
        probe = __builtin_fmaf(x2, x3, probe);
        eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
        eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
    }
    if (__builtin_amdgcn_classf(probe, kSpecial)) {
#pragma unroll
        for (int j = 0; j < R * 4; ++j) eb[j] = __float_as_uint(sf(__uint_as_float(eb[j])));
    }
    if (p.e_bits) {
        // diagnostics: e of every token in the row's frame, dead tokens as 0
        uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
        auto live = [&](uint32_t xb) { const uint32_t b = e_bits_raw(__uint_as_float(xb), M); return b < kEMinBits || b > 0x3FFFFFFFu ? 0u : b; };
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) dst[base4 + j * kThreads] = make_uint4(live(eb[j * 4]), live(eb[j * 4 + 1]), live(eb[j * 4 + 2]), live(eb[j * 4 + 3]));
    }
    if (skip) return;
    // The tokens of the boundary bin, found by two comparisons on x, go into this wave's queue: the lanes
    // that hold one write side by side (a prefix count of the wave's vote gives each its place).  Only
    // they need their e, in the dense loops below.
    uint32_t qfill = 0;                                  // wave-uniform: every lane takes part in every vote
#pragma unroll
    for (int j = 0; j < R; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float x = __uint_as_float(eb[j * 4 + q]);
            const bool in = j < nv && x >= x_lo && x < x_hi;
            const uint64_t vote = __ballot(in);
            if (in) {
                const uint32_t pos = qfill + __builtin_amdgcn_mbcnt_hi((uint32_t)(vote >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)vote, 0u));
                if (pos < (uint32_t)kQ) { s.qx[wave][pos] = eb[j * 4 + q]; s.qi[wave][pos] = (uint16_t)((j * 4 + q) * NT + tid); }
            }
            qfill += (uint32_t)__popcll(vote);
        }
    }
    if (lane == 0 && qfill > (uint32_t)kQ) s.over = 1u;
    __syncthreads();
    // Some wave holds more tokens of the bin than its queue (a bin with a quarter of the row and more: very
    // flat rows at a high temperature, rows of few distinct values): the slice is then gone through
    // again from memory, which has just been read -- fn(bits of e, token index) for the bin's tokens.
    const bool over = s.over != 0u;
    auto place = [&](uint32_t id) { const uint32_t jq = id / NT, t = id - jq * NT; return (base4 - (uint32_t)tid + t + (jq >> 2) * NT) * 4u + (jq & 3u); };
    auto bin_tokens_again = [&](auto fn) {
        constexpr int kAhead = 4;
#pragma unroll 1
        for (int j0 = 0; j0 < R; j0 += kAhead) {
            float4 l[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) l[u] = load_logits4(lrow, min(base4 + (uint32_t)(j0 + u) * kThreads, V4 - 1u), DT);
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                if (j0 + u < nv) {
                    const uint32_t i4 = base4 + (uint32_t)(j0 + u) * kThreads;
                    const float x4[4] = {sf(l[u].x * p.c), sf(l[u].y * p.c), sf(l[u].z * p.c), sf(l[u].w * p.c)};
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (x4[q] >= x_lo && x4[q] < x_hi) fn(e_bits_raw(x4[q], M), i4 * 4u + (uint32_t)q);
                }
            }
        }
    };
    auto count_one = [&](uint32_t b) {
        atomicAdd(reinterpret_cast<unsigned long long *>(&s.sub[((b >> 14) & 127u) * kWideRep + (lane & (kWideRep - 1))]),
                  (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
    };
    if (!over) {
        // four queue entries per lane and round: their LDS round trips overlap
        for (uint32_t i0 = 0; i0 < qfill; i0 += 4 * kWave) {
            uint32_t xs[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) xs[u] = s.qx[wave][min(i0 + (uint32_t)(u * kWave + lane), (uint32_t)kQ - 1u)];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = i0 + (uint32_t)(u * kWave + lane);
                if (i < qfill) {
                    const uint32_t b = e_bits_raw(__uint_as_float(xs[u]), M);
                    s.qx[wave][i] = b;
                    count_one(b);
                }
            }
        }
    } else {
        bin_tokens_again([&](uint32_t b, uint32_t) { count_one(b); });
    }
    __syncthreads();

    if (wave == 0) {
        // The slice's sub-bins as running sums from the top, kept under the slice's name (the finishing
        // workgroup adds the slices' up).  Lane l owns sub-bins 127 - 2l and 126 - 2l; packed sums never
        // carry from one field into the other.
        uint64_t w0 = 0, w1 = 0;
#pragma unroll
        for (int c = 0; c < kWideRep; ++c) { w0 += s.sub[(127 - 2 * lane) * kWideRep + c]; w1 += s.sub[(126 - 2 * lane) * kWideRep + c]; }
        const uint64_t inc = wave_inclusive_scan(w0 + w1);
        const uint64_t c_hi = inc - w1, c_lo = inc;     // at 127 - 2l, 126 - 2l
        s.cp[127 - 2 * lane] = c_hi; s.cp[126 - 2 * lane] = c_lo;
        st[2 + 127 - 2 * lane] = c_hi; st[2 + 126 - 2 * lane] = c_lo;
        if (lane == 0) { s.cp[128] = 0; s.cp[129] = 0; st[2 + 128] = 0; }
        // Where this slice expects the row's threshold: the first sub-bin from the top at which its own
        // running count or mass, scaled to the row's share of the bin, reaches what the row still needs.
        // Only a guess (it decides what is set aside, nothing else): the masses in rounded arithmetic.
        const uint32_t n_s = pack_count(lane63(inc));
        const uint64_t cb = pl->cnt_bin;
        const uint64_t need_k = (uint64_t)p.top_k - (uint64_t)pl->cnt_above;
        const float need_f = pl->need_mf * (float)n_s, cb_f = (float)pl->cnt_bin;
        auto enough = [&](uint64_t x) {
            const float units = (float)pack_count(x) * 8388608.0f + (float)(x & kPackMask);
            return (uint64_t)pack_count(x) * cb >= need_k * (uint64_t)n_s || units * cb_f >= need_f;
        };
        const uint32_t cand = enough(c_hi) ? 128u - 2u * (uint32_t)lane : enough(c_lo) ? 127u - 2u * (uint32_t)lane : 0u;   // sub-bin + 1
        const uint32_t jp1 = wave_max_u32(cand);
        const int j_est = jp1 ? (int)jp1 - 1 : 0;
        // the widest window around it that fits: lane l tries half-widths l and l + 64
        auto inside = [&](int w) {
            const int lo = max(0, j_est - w), hi = min(127, j_est + w);
            return pack_count(s.cp[lo]) - pack_count(s.cp[hi + 1]);
        };
        // How much to set aside: the slice's running count at the row's threshold differs from its share by
        // about the square root of that count when the slice is a fair sample of the row -- at most
        // sqrt(n_s) tokens; six times that either side, at least 64 tokens, and no more than fits.  (What
        // is set aside is written out and read again: the whole bin would cost a fifth of the pass.)
        const uint32_t room = min((uint32_t)kWideCap, max(64u, (uint32_t)(12.0f * __builtin_sqrtf((float)n_s))));
        const uint64_t fit0 = __ballot(inside(lane) <= room), fit1 = __ballot(inside(lane + 64) <= room);
        const int nfit = __popcll(fit0) + __popcll(fit1);       // counts grow with the width: the fitting widths are a prefix
        uint32_t wl = 1u, wh = 0u, wn = 0u;
        if (n_s != 0u && nfit != 0) {
            const int w = nfit - 1;
            wl = (uint32_t)max(0, j_est - w); wh = (uint32_t)min(127, j_est + w);
            wn = inside(w);
        }
        // where each sub-bin of the window begins among the tokens set aside (largest values first)
        const uint32_t top = pack_count(s.cp[min(wh, 127u) + 1]);
        s.off[127 - 2 * lane] = pack_count(s.cp[128 - 2 * lane]) - top;
        s.off[126 - 2 * lane] = pack_count(c_hi) - top;
        if (lane == 0) {
            s.win_lo = wl; s.win_hi = wh; s.n = wn;
            PartHdr *ph = &v.hdr[(size_t)row * G + part];
            ph->cov = wl | wh << 8 | kWideValid;
            ph->n = wn;
        }
    } else if (wave == 1) {
        // kept mass of this slice above the boundary bin, from the bins the first pass kept under the
        // slice's name (slice frame: bin t is the row's bin t - 4 delta)
        const float dd = M - __builtin_floorf(fkey_inv(own_key));
        const uint32_t delta = dd >= 64.0f ? 64u : (uint32_t)dd;
        const int rb = (int)(b1 - kBin0);
        u128 ms = 0;
        if (delta < 41u) {
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int t = kSB - 1 - 3 * lane - i;
                const int ri = t - 4 * (int)delta;
                if (t >= 0 && ri > rb && own_bins[i]) ms += pack_mass(own_bins[i], (kBin0 + (uint32_t)ri) >> 2);
            }
        }
        const u128 tot = wave_sum(ms);
        if (lane == 0) { st[0] = (uint64_t)tot; st[1] = (uint64_t)(tot >> 64); }
    }
    __syncthreads();
    const uint32_t win_lo = s.win_lo, win_hi = s.win_hi, n = s.n;
    auto set_aside = [&](uint32_t b, uint32_t idx) {
        const uint32_t sb = (b >> 14) & 127u;
        if (sb >= win_lo && sb <= win_hi) {
            const uint32_t slot = atomicAdd(&s.off[sb], 1u);
            if (slot < (uint32_t)kWideCap) s.stage[slot] = ((uint64_t)b << 32) | idx;
        }
    };
    if (!over) {
        for (uint32_t i0 = 0; i0 < qfill; i0 += 4 * kWave) {
            uint32_t bs[4], ids[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t i = min(i0 + (uint32_t)(u * kWave + lane), (uint32_t)kQ - 1u);
                bs[u] = s.qx[wave][i]; ids[u] = s.qi[wave][i];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (i0 + (uint32_t)(u * kWave + lane) < qfill) set_aside(bs[u], place(ids[u]));
        }
    } else {
        bin_tokens_again(set_aside);
    }
    __syncthreads();
    for (uint32_t i = (uint32_t)tid; i < min(n, (uint32_t)kWideCap); i += kThreads) st[kWideHead + i] = s.stage[i];
}

template <int SLICE_LOG2>
__device__ __forceinline__ void wide_finish_row(const Params &p, const StreamView &v, Lds &s, LdsB &t, const uint32_t row)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const PartHdr *hdrs = v.hdr + (size_t)row * G;
    RowCtl *rc = p.ctl_end - 1 - row;

    if (tid == 0) { s.abort = 0; s.host_words = p.host_words; t.fail = 0; t.result = 0u; }
    PartHdr ph;
    ph.mkey = 0; ph.cov = 0; ph.n = 0; ph.cut = 0;
    if ((uint32_t)tid < G) ph = hdrs[tid];
    // the row's level 2: a thread sums half of the slices' running sums at one of the 128 sub-bin edges (the
    // 129th is zero by definition; a load instruction reads one slice's consecutive words, sixteen slices'
    // loads in flight at a time); the row's sub-bin j is the difference of two neighbours
    uint64_t cpsum = 0;
    {
        const uint32_t edge = (uint32_t)tid & 127u, upper = (uint32_t)tid >> 7;
        const uint32_t g_mid = (G + 1u) >> 1, g_hi = upper ? G : g_mid;
        const uint64_t *cp0 = v.stash + (size_t)row * G * kStashCap + 2 + edge;
        for (uint32_t g0 = upper ? g_mid : 0u; g0 < g_hi; g0 += 16u) {
            uint64_t w[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) w[u] = cp0[(size_t)min(g0 + (uint32_t)u, G - 1u) * kStashCap];
#pragma unroll
            for (int u = 0; u < 16; ++u) if (g0 + (uint32_t)u < g_hi) cpsum += w[u];
        }
    }
    WidePlan *plan = reinterpret_cast<WidePlan *>(rc->A);
    const WidePlan pl = *plan;
    const bool drawer = tid == kWave && !p.inj_u;
    if (drawer) {
        uint32_t *rng_st = p.rng + (size_t)row * 16;
        uint32_t rs[6], o[4];
#pragma unroll
        for (int i = 0; i < 6; ++i) rs[i] = rng_st[i];
        philox4x32_10(rs[2], rs[3], rs[4], rs[5], rs[0], rs[1], o);
        t.rand64 = ((uint64_t)o[0] << 32) | o[1];
        rng_st[2] = rs[2] + 1u;                          // the row is finished here whatever happens
        if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
    }
    __syncthreads();                                     // everyone holds the plan: its words can go back to zero
    if (tid < (int)(sizeof(WidePlan) / sizeof(uint64_t))) rc->A[tid] = 0;
    const float xmax = fkey_inv(pl.kmax);
    const float M = __builtin_floorf(xmax);
    const uint64_t top_k = (uint64_t)p.top_k;
    Found f;
    f.bin = pl.b1; f.cnt_above = pl.cnt_above; f.cnt_bin = pl.cnt_bin; f.pad = 0; f.local_above = 0;
    f.mass_above = (u128)pl.mass_above[0] | ((u128)pl.mass_above[1] << 64);
    const u128 D = (u128)pl.D[0] | ((u128)pl.D[1] << 64), P = (u128)pl.P[0] | ((u128)pl.P[1] << 64);
    if (tid == 0) { s.D = D; s.P = P; }
    const uint32_t exb = f.bin >> 2;
    const uint64_t rand64 = p.inj_u ? 0ull : t.rand64;

    auto tell_policy = [&]() {
        if (tid == 0) {
            const uint32_t c = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
            if (c == 0u && p.host_words)
                __hip_atomic_store(p.host_words + p.report, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    };
    auto slow = [&]() {
        finish_row_slow(p, s, t, row, xmax, rand64);
        if (tid == 0) {
            const uint32_t c = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
            if (c == 0u && p.host_words)                 // the call's first such row tells the caller's policy at once
                __hip_atomic_store(p.host_words + p.report, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    };

    // one tie of all the row's tokens: as on the streaming path
    if (pl.skip) {
        if (tid == 0) {
            const uint32_t thr1 = e_bits_of(xmax, M);
            const Target tg = tie_and_target(p, row, rand64, xmax, D, P, thr1, 0u, f.cnt_bin, (u128)0, 0u, true);
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

    // level 2: the row's sub-bins of the boundary bin must add up to the bin
    const uint32_t b1 = f.bin;
    if (tid >= 128) s.g[tid] = cpsum;                    // the upper half of the slices, beside the lower half's place
    __syncthreads();
    if (tid < 128) s.g[tid] = cpsum + s.g[tid + 128];
    __syncthreads();
    if (tid == 128) s.g[128] = 0;
    __syncthreads();
    if (tid < 128) s.hm[tid] = s.g[tid] - s.g[tid + 1];
    const uint32_t cnt2 = pack_count(s.g[0]);
    __syncthreads();
    if (cnt2 != f.cnt_bin) return slow();
    f = hist_find128(s, s.hm, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
    const uint32_t b2 = f.bin;

    // what every slice has of that sub-bin, and whether the window it set aside covers it
    uint32_t mine = 0, offs = 0;
    u128 kept_g = 0;                                     // kept weight of slice tid, so far without its listed tokens
    bool bad = false;
    if ((uint32_t)tid < G) {
        const uint64_t *st = v.stash + ((size_t)row * G + tid) * kStashCap;
        if (!(ph.cov & kWideValid)) bad = true;
        else {
            const uint32_t wl = ph.cov & 255u, wh = (ph.cov >> 8) & 255u;
            const uint64_t c_hi = st[2 + b2 + 1], c_lo = st[2 + b2];
            mine = pack_count(c_lo) - pack_count(c_hi);
            if (mine) {
                if (b2 < wl || b2 > wh) bad = true;
                else offs = pack_count(c_hi) - pack_count(st[2 + wh + 1]);
            }
            kept_g = ((u128)st[0] | ((u128)st[1] << 64)) + (c_hi ? pack_mass(c_hi, exb) : (u128)0);
        }
    }
    if (bad) t.fail = 1;
    {
        uint32_t inc = wave_inclusive_scan(mine);
        __syncthreads();
        if (lane == kWave - 1) s.u32[wave] = inc;
        __syncthreads();
        for (int w = 0; w < wave; ++w) inc += s.u32[w];
        t.take[tid] = inc;
        t.m4[tid] = offs;
        __syncthreads();
    }
    const uint32_t total = t.take[kThreads - 1];
    if (t.fail || total != f.cnt_bin || total > v.list_cap) return slow();

    // gather: entry i belongs to the first slice whose inclusive prefix exceeds i; a thread takes a run
    {
        const uint32_t per = (total + kThreads - 1u) / kThreads;
        uint32_t i = (uint32_t)tid * per;
        const uint32_t iend = min(total, i + per);
        if (i < iend) {
            uint32_t lo_g = 0, hi_g = G - 1;
            while (lo_g < hi_g) {
                const uint32_t mid = (lo_g + hi_g) >> 1;
                if (t.take[mid] > i) hi_g = mid; else lo_g = mid + 1;
            }
            uint32_t g = lo_g, gbase = g ? t.take[g - 1] : 0u, gend = t.take[g];
            for (; i < iend; ++i) {
                while (i >= gend) { ++g; gbase = gend; gend = t.take[g]; }
                t.list[i] = v.stash[((size_t)row * G + g) * kStashCap + kWideHead + t.m4[g] + (i - gbase)];
            }
        }
    }
    __syncthreads();

    // the remaining 14 bits of the threshold, on the listed tokens (all of them lie in the sub-bin)
    uint32_t lo = (b1 << 21) | (b2 << 14), span = (1u << 14) - 1u;
    for (uint32_t lv = 3; lv <= (uint32_t)kLevels && f.cnt_bin > 1u; ++lv) {
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
    if (tid == 0) {
        const Target tg = tie_and_target(p, row, rand64, xmax, D, P, thr, f.cnt_above, f.cnt_bin, f.mass_above, 7u, true);
        s.bc64[1] = tg.w_tie; s.bc128[0] = tg.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    const u128 r = s.bc128[0];
    // as a probe for the streaming path: would this row's kept set have fitted the stashes of an attempt?
    if (p.probe && f.cnt_above + f.cnt_bin > 512u) tell_policy();
    auto weight = [=](uint32_t b) -> uint64_t { return (b > thr) ? w_of_bits(b) : (b == thr ? w_tie : 0ull); };

    // kept weight per slice: the listed tokens of slice g are entries [take[g-1], take[g])
    if ((uint32_t)tid < G) {
        const uint32_t a = tid ? t.take[tid - 1] : 0u, e = t.take[tid];
        for (uint32_t i = a; i < e; ++i) kept_g += weight((uint32_t)(t.list[i] >> 32));
    }
    u128 inc = wave_inclusive_scan(kept_g);
    __syncthreads();
    if (lane == kWave - 1) s.q128[wave] = inc;
    __syncthreads();
    for (int w = 0; w < wave; ++w) inc += s.q128[w];
    const u128 exc = inc - kept_g;
    if (exc < r && r <= inc) { t.bucket = (uint32_t)tid; s.bc128[1] = r - exc; }
    __syncthreads();
    const uint32_t g = t.bucket;
    const u128 r_in = s.bc128[1];
    __syncthreads();
    keep_pick<SLICE_LOG2>(p, s, t, row, M, g << SLICE_LOG2, r_in, weight);
}

template <int SLICE_LOG2>
__global__ void __launch_bounds__(kThreads) wide_finish_kernel(const Params p, const StreamView v)
{
    __shared__ Lds s;
    __shared__ LdsB t;
    extern __shared__ __align__(16) unsigned char finish_dyn[];
    t.list = reinterpret_cast<uint64_t *>(finish_dyn);
    wide_finish_row<SLICE_LOG2>(p, v, s, t, blockIdx.x);
}

}  // namespace rs
