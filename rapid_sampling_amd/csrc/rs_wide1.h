// The wide path in one pass over the logits: kept sets of thousands of tokens, the logits read once
// plus a sample of them.
//
//   wide_sample_kernel   one workgroup per row over a SAMPLE of the row (chunks of 256 tokens spread
//                        evenly over it, an eighth of the row and at most 32768 tokens, kept in
//                        registers): the sample's frame, its level-1 histogram, the bin in which its
//                        kept set becomes sufficient, and from the sampling error of that rank a RANGE
//                        of 1, 2, 4 or 8 level-1 bins that should hold the row's threshold, the range's
//                        128 sub-bins counted on the sample, and the WINDOW of sub-bins around the
//                        expected threshold that the slices are to set aside.  A guess: it decides what
//                        is counted finely and what is set aside, nothing else.
//   wide1_kernel         one workgroup per slice, the only pass over all the logits: the slice's frame
//                        and level-1 histogram as in the streaming pass (added to the row's), and at
//                        the same time its tokens of the range by sub-bin.  Left under the slice's name:
//                        running counts and masses of the range from its top, the mass above the range,
//                        and the window's tokens ordered by sub-bin.  Masses and bit patterns are
//                        written relative to the range's top octave, which is the same for every slice
//                        whatever its own frame.
//   wide1_finish_kernel  one workgroup per row: the row's frame and exact level-1 boundary from the
//                        row's histogram; if that boundary lies in the range, the row's running sums
//                        (the slices' added up) give the boundary sub-bin exactly, its tokens come from
//                        the slices' windows, the remaining bits of the threshold are resolved on them,
//                        and the slice that holds the target follows from per-slice kept weights, as on
//                        the two-pass wide path.  A row whose threshold the range or some slice's
//                        window does not cover (a sample that is no fair picture of the row: a few
//                        tokens that carry most of the mass) is done the slow way and reported.
// Same integers as every other path.
#pragma once

#include "rs_wide.h"

namespace rs {

constexpr int      kW1Head    = 260;                     // words at the head of a slice's stash region: mass above the range (2), running masses (129 x 2)
constexpr int      kW1Cap     = kStashCap - kW1Head;     // tokens a slice can set aside
constexpr int      kW1Rep     = 4;                       // copies of each sub-bin while it is counted
constexpr int      kW1SampleT = 1024;                    // threads of the sampling kernel
constexpr int      kW1SampleR = 8;                       // groups of four tokens per thread of the sampling kernel: 32768 tokens at most
constexpr uint32_t kW1Rounds  = 9u;                      // DiagRow::rounds of a row finished here

// What the sampling kernel leaves for a row (in the first words of RowCtl::A; the finishing workgroup
// puts them back to zero).
struct WideGuess {
    uint32_t state;           // 1: range and window below; 2: no guess (the finishing workgroup does the row alone)
    float    M;               // the sample's frame: floor of its largest x
    uint32_t bin_top;         // top level-1 bin of the range, in the sample's frame
    uint32_t n_log2;          // the range is 2^n_log2 bins, bin_top downwards; its 128 sub-bins are 2^(14 + n_log2) bit patterns each
    uint32_t j_lo, j_hi;      // the window: sub-bins of the range whose tokens the slices set aside
    uint32_t j_est;           // where the threshold is expected (what a slice keeps when the window does not fit)
    uint32_t pad;
};
static_assert(sizeof(WideGuess) % sizeof(uint64_t) == 0 && sizeof(WideGuess) <= sizeof(uint64_t) * 2 * kMaxParts, "fits RowCtl::A");

struct LdsS {                         // sampling kernel
    u128     D, P;
    Found    found;
    uint64_t g[kNB];                  // the sample's level-1 histogram, sample frame
    uint64_t hm[kNB * 8];             // the same while it is counted: eight copies of each bin (lane l adds to copy l % 8)
    uint32_t sub[128 * 4];            // the range's sub-bins, counts only, four copies
    uint32_t u32[16];
    uint32_t b32[8];
};

__device__ __forceinline__ float f_of_u128(u128 x)
{
    return (float)(uint64_t)(x >> 64) * 18446744073709551616.0f + (float)(uint64_t)x;
}

// The range in a frame M2 given in the frame M1: bins move by 4 per octave.  Frames further apart than
// 64 octaves are treated as 64 apart (nothing of such a slice lies in the range either way).
__device__ __forceinline__ int range_top_in_frame(uint32_t bin_top, float M_from, float M_to)
{
    const float d = fminf(fmaxf(M_from - M_to, -64.0f), 64.0f);
    return (int)bin_top + 4 * (int)d;
}

__global__ void __launch_bounds__(kW1SampleT) wide_sample_kernel(const Params p, const StreamView v)
{
    constexpr int kThreads = kW1SampleT;                 // (shadows the namespace's: this kernel's workgroup size)
    __shared__ LdsS s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t row = blockIdx.x;
    RowCtl *rc = p.ctl_end - 1 - row;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    // chunks of 64 groups (256 tokens, 1 KiB of fp32): every S-th one, from the middle of its stretch -- an
    // eighth of a long row, more of a short one, 32768 tokens at most
    const uint32_t S = max(max(((uint32_t)p.V + 32767u) >> 15, min(8u, (uint32_t)p.V >> 14)), 1u);
    const uint32_t nch = (V4 >> 6) / S;                  // <= 128
    const uint32_t ng = nch * 64u;                       // sampled groups, <= 8192
    const uint32_t n_s = ng * 4u;
    const char *lrow = logits_row(p, row);
    if (nch == 0u) {                                     // a row of fewer than 256 tokens: nothing to go by
        WideGuess *none = reinterpret_cast<WideGuess *>(rc->A);
        if (tid == 0) { none->state = 2u; none->M = 0.0f; none->bin_top = kTop1; none->n_log2 = 0u; none->j_lo = 1u; none->j_hi = 0u; none->j_est = 0u; none->pad = 0u; }
        return;
    }
    for (int i = tid; i < kNB * 8; i += kThreads) s.hm[i] = 0;
    for (int i = tid; i < 128 * 4; i += kThreads) s.sub[i] = 0;

    uint32_t eb[kW1SampleR * 4];
    float lmax = -3.402823466e+38f;
#pragma unroll
    for (int j = 0; j < kW1SampleR; ++j) {
        const uint32_t g = (uint32_t)tid + (uint32_t)j * kThreads;
        const uint32_t src = ((g >> 6) * S + (S >> 1)) * 64u + (g & 63u);
        const float4 l = load_logits4(lrow, g < ng ? src : 0u, p.dtype);
        const float x0 = sf(l.x * p.c), x1 = sf(l.y * p.c), x2 = sf(l.z * p.c), x3 = sf(l.w * p.c);
        if (g < ng) lmax = fmaxf(lmax, fmaxf(fmaxf(x0, x1), fmaxf(x2, x3)));
        eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
        eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
    }
    uint32_t kmax = wave_max_u32(fkey(lmax));
    if (lane == 0) s.u32[wave] = kmax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kThreads / kWave; ++w) kmax = max(kmax, s.u32[w]);
    static_assert(kW1SampleT / kWave <= 16, "LdsS::u32");
    const float M = __builtin_floorf(fkey_inv(kmax));
    // e in the sample's frame; live tokens into the histogram
#pragma unroll
    for (int j = 0; j < kW1SampleR; ++j) {
        const bool in = (uint32_t)tid + (uint32_t)j * kThreads < ng;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t b = in ? e_bits_raw(__uint_as_float(eb[j * 4 + q]), M) : 0u;
            eb[j * 4 + q] = b;
            if (b >= kEMinBits)
                atomicAdd(reinterpret_cast<unsigned long long *>(&s.hm[(b >> 21) * 8u + (uint32_t)(lane & 7)]),
                          (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
        }
    }
    __syncthreads();
    for (int b = tid; b < kNB; b += kThreads)
        s.g[b] = b >= (int)kBin0 ? s.hm[b * 8] + s.hm[b * 8 + 1] + s.hm[b * 8 + 2] + s.hm[b * 8 + 3] +
                                   s.hm[b * 8 + 4] + s.hm[b * 8 + 5] + s.hm[b * 8 + 6] + s.hm[b * 8 + 7] : 0ull;
    __syncthreads();
    // the sample's share of top_k
    const uint64_t k_s = p.top_k >= p.V ? (uint64_t)n_s : ((uint64_t)p.top_k * n_s + (uint64_t)p.V - 1u) / (uint64_t)p.V;
    const Found f = hist_find_level1<false, false, LdsS>(s, max(k_s, (uint64_t)1), p.top_p, lane, wave);
    // A sample that is one tie (rows of equal logits) says nothing about a threshold, and a range around it
    // would queue every token of the row up at one sub-bin: no guess.  (A row that is one tie of all its
    // tokens is recognised by the finishing workgroup from the row's bins alone.)
    if (f.cnt_bin == n_s && bin_is_one_tie(s.g[f.bin], f.bin, e_bits_of(fkey_inv(kmax), M))) {
        WideGuess *none = reinterpret_cast<WideGuess *>(rc->A);
        if (tid == 0) { none->state = 2u; none->M = M; none->bin_top = kTop1; none->n_log2 = 0u; none->j_lo = 1u; none->j_hi = 0u; none->j_est = 0u; none->pad = 0u; }
        return;
    }

    // How many of the sample's tokens lie above its threshold, roughly (the position inside the boundary
    // bin by linear interpolation of count and mass), and how far off that rank may be for the row:
    // the binomial error of a rank in a sample, doubled for what the sample does not know about the
    // row's total mass, six times that either side.
    const float cnt_bin = (float)f.cnt_bin, cnt_above = (float)f.cnt_above;
    const u128 mass_bin = pack_mass(s.g[f.bin], f.bin >> 2);
    const float fc = ((float)k_s - cnt_above) / fmaxf(cnt_bin, 1.0f);
    const float fm = f_of_u128(s.P - f.mass_above) / fmaxf(f_of_u128(mass_bin), 1.0f);
    const float fr = fminf(fminf(fc, fm), 1.0f);
    const float k_eff = cnt_above + fr * cnt_bin;
    const float sd = __builtin_sqrtf(fmaxf(4.0f, k_eff * (1.0f - k_eff / (float)n_s)));
    const float marg = 12.0f * sd + 8.0f;
    if (wave == 0) {
        // level-1 bins in which the ranks k_eff -+ marg lie (ranks count from the largest token)
        uint32_t c3[3], cs = 0;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int idx = (int)kTop1 - 3 * lane - i;
            c3[i] = idx >= (int)kBin0 ? pack_count(s.g[idx]) : 0u;
            cs += c3[i];
        }
        const uint32_t ci = wave_inclusive_scan(cs);
        const uint32_t total = lane63(ci);
        const uint32_t t_hi = (uint32_t)fmaxf(1.0f, __builtin_floorf(k_eff - marg));
        const uint32_t t_lo = (uint32_t)fminf((float)total, __builtin_ceilf(k_eff + marg));
        uint32_t run = ci - cs;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const uint32_t nx = run + c3[i];
            const uint32_t bin = kTop1 - (uint32_t)(3 * lane + i);
            if (run < t_hi && nx >= t_hi) { s.b32[0] = bin; s.b32[2] = run; }      // top bin of the range, tokens above it
            if (run < t_lo && nx >= t_lo) s.b32[1] = bin;                           // its lowest bin
            run = nx;
        }
    }
    __syncthreads();
    const uint32_t bin_top = s.b32[0], bin_bot = s.b32[1], cnt_ar = s.b32[2];
    const uint32_t span_bins = bin_top - bin_bot + 1u;
    const uint32_t n_log2 = span_bins <= 1u ? 0u : 32u - (uint32_t)__builtin_clz(span_bins - 1u);
    WideGuess *gs = reinterpret_cast<WideGuess *>(rc->A);
    if (n_log2 > 3u) {
        if (tid == 0) { gs->state = 2u; gs->M = M; gs->bin_top = bin_top; gs->n_log2 = 0u; gs->j_lo = 1u; gs->j_hi = 0u; gs->j_est = 0u; gs->pad = 0u; }
        return;
    }
    // the range's sub-bins on the sample (counts), and the window from the same ranks
    const uint32_t sh = 14u + n_log2;
    const uint32_t lo_bits = (bin_top + 1u - (1u << n_log2)) << 21;
    const uint32_t lo_live = max(lo_bits, kEMinBits), width = ((bin_top + 1u) << 21) - lo_live;
#pragma unroll
    for (int j = 0; j < kW1SampleR; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t b = eb[j * 4 + q];
            if (b - lo_live < width) atomicAdd(&s.sub[((b - lo_bits) >> sh) * 4u + (uint32_t)(lane & 3)], 1u);
        }
    __syncthreads();
    if (wave == 0) {
        auto cnt_of = [&](int j) { return s.sub[j * 4] + s.sub[j * 4 + 1] + s.sub[j * 4 + 2] + s.sub[j * 4 + 3]; };
        const uint32_t c0 = cnt_of(127 - 2 * lane), c1 = cnt_of(126 - 2 * lane);
        const uint32_t ci = wave_inclusive_scan(c0 + c1);
        const uint32_t total = cnt_ar + lane63(ci);
        const uint32_t rc_hi = cnt_ar + ci - c1, rc_lo = cnt_ar + ci;              // tokens at or above sub-bin 127 - 2l, 126 - 2l
        // sub-bin in which rank r lies: the highest one at or above which r tokens lie
        auto sub_of = [&](uint32_t r) {
            const uint32_t cand = rc_hi >= r ? 128u - 2u * (uint32_t)lane : rc_lo >= r ? 127u - 2u * (uint32_t)lane : 0u;    // sub-bin + 1
            const uint32_t m = wave_max_u32(cand);
            return m ? m - 1u : 0u;
        };
        const uint32_t t_hi = (uint32_t)fmaxf(1.0f, __builtin_floorf(k_eff - marg));
        const uint32_t t_lo = (uint32_t)fminf((float)total, __builtin_ceilf(k_eff + marg));
        const uint32_t t_mid = (uint32_t)fminf((float)total, fmaxf(1.0f, k_eff));
        const uint32_t j_hi = t_hi <= cnt_ar ? 127u : sub_of(t_hi), j_lo = sub_of(t_lo), j_est = sub_of(t_mid);
        if (lane == 0) {
            gs->state = 1u; gs->M = M; gs->bin_top = bin_top; gs->n_log2 = n_log2;
            gs->j_lo = j_lo; gs->j_hi = max(j_hi, j_lo); gs->j_est = min(max(j_est, j_lo), max(j_hi, j_lo)); gs->pad = 0u;
        }
    }
}

template <int kRep>
struct LdsW1 {
    union {
        uint64_t hm[kNB * kRep];      // the slice's bins by bits >> 21
        uint64_t stage[kW1Cap];       // then: the tokens set aside, ordered by sub-bin, before they are written out
    };
    uint64_t sub[128 * kW1Rep];       // the slice's tokens of the range by sub-bin
    uint32_t cpc[130];                // tokens of the slice in the range at or above sub-bin j; [128] = [129] = 0
    uint32_t off[128];                // where the next token of sub-bin j goes
    uint32_t u32[16];
    uint32_t win_lo, win_hi, n;
};

template <int R, int DT>              // 256 threads, each with R groups of four tokens of the slice; DT the logits' type
__global__ void __launch_bounds__(kThreads, (R <= 8 ? 5 : RS_STREAM_WAVES)) wide1_kernel(const Params p, const StreamView v)
{
    constexpr int kRep = stream_copies<R>();
    constexpr int NT = kThreads;
    __shared__ LdsW1<kRep> s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const uint32_t row = blockIdx.x / G, part = blockIdx.x - row * G;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t base4 = part * (uint32_t)(NT * R) + (uint32_t)tid;
    const int nv = base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - base4 + NT - 1) / NT);
    const char *lrow = logits_row(p, row);
    RowCtl *rc = p.ctl_end - 1 - row;
    uint64_t *st = v.stash + ((size_t)row * G + part) * kStashCap;

    const bool reporter = blockIdx.x == 0 && tid == 0;
    PrevCall prev;
    prev.slow_rows = 0; prev.meta = 0;
    if (reporter) prev = report_begin(p);
    uint32_t eb[R * 4];                                 // l, then x, then bits(e)
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
    const WideGuess gs = *reinterpret_cast<const WideGuess *>(rc->A);
    {
        uint4 *z = reinterpret_cast<uint4 *>(s.hm);
#pragma unroll
        for (int i = 0; i < kNB * kRep / 2 / NT; ++i) z[tid + i * NT] = make_uint4(0u, 0u, 0u, 0u);
        static_assert(kNB * kRep % (2 * NT) == 0, "whole stores");
        for (int i = tid; i < 128 * kW1Rep; i += NT) s.sub[i] = 0;
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
    if (reporter) report_end(p, prev, true);

    uint32_t k = wave_max_u32(fkey(lmax));
    if (lane == 0) s.u32[wave] = k;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < (NT / kWave); ++w) k = max(k, s.u32[w]);
    const float M = __builtin_floorf(fkey_inv(k));

    // The range in this slice's frame.  A range whose top lies more than 40 octaves below the slice's
    // largest token is dead in the row's frame, whatever the sample made of it: such a slice says
    // nothing (the row is then done the slow way).
    const int bt = range_top_in_frame(gs.bin_top, gs.M, M);
    const bool ranged = gs.state == 1u && bt >= (int)kBin0;
    const uint32_t sh = 14u + gs.n_log2;
    const uint32_t lo_bits = (uint32_t)(bt + 1 - (1 << gs.n_log2)) << 21;
    const uint32_t lo_live = max(lo_bits, kEMinBits);
    const uint32_t width = ranged ? ((uint32_t)(bt + 1) << 21) - lo_live : 0u;          // no pattern is this far above lo_live when the range is off
    const uint32_t exb_top = (uint32_t)bt >> 2;

    // e in the slice's frame (not clamped at 2^-40) and ONE histogram atomic per token, as in the streaming
    // pass: a token of the range is counted in its sub-bin, every other token in its level-1 bin -- the
    // address is selected, nothing is branched on (a conditional per token keeps the compiler from
    // interleaving the tokens' polynomials and is issued whenever some lane of the wave takes it).  Slots
    // past the end of the row become 0.
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (j < nv) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t b = e_bits_raw(__uint_as_float(eb[j * 4 + q]), M);
                eb[j * 4 + q] = b;
                uint64_t *bin = &s.hm[(b >> 21) * kRep + (lane & (kRep - 1))];
                uint64_t *sub = &s.sub[(((b - lo_bits) >> sh) & 127u) * kW1Rep + (lane & (kW1Rep - 1))];
                atomicAdd(reinterpret_cast<unsigned long long *>(b - lo_live < width ? sub : bin),
                          (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
            }
        } else {
            eb[j * 4] = 0; eb[j * 4 + 1] = 0; eb[j * 4 + 2] = 0; eb[j * 4 + 3] = 0;
        }
    }
    __syncthreads();
    // the range's level-1 bins: their sub-bins added up (everything behind this reads the bins as the
    // streaming pass does)
    if (ranged && tid < 128) {
        uint64_t w = 0;
#pragma unroll
        for (int c = 0; c < kW1Rep; ++c) w += s.sub[tid * kW1Rep + c];
        if (w) atomicAdd(reinterpret_cast<unsigned long long *>(&s.hm[((lo_bits + ((uint32_t)tid << sh)) >> 21) * kRep + (tid & (kRep - 1))]),
                         (unsigned long long)w);
    }
    if (p.e_bits) {
        // diagnostics: e of every token, still in the slice's frame; the finishing workgroup re-bases it
        uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) dst[base4 + j * NT] = make_uint4(eb[j * 4], eb[j * 4 + 1], eb[j * 4 + 2], eb[j * 4 + 3]);
    }
    __syncthreads();
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
    // the slice's live bins, added to the row's by absolute octave and kept under the slice's name (as in the streaming pass)
    if (tid < kSB) {
        const uint64_t w = bin_total(tid);
        const float mm = M - 128.0f * __builtin_floorf(M * 0.0078125f);
        v.shist[((size_t)row * G + part) * kSB + tid] = w;
        if (w) a_add(&rc->rowhist[((uint32_t)(int)mm * 4u + (uint32_t)tid - 160u) & 511u], w);
    }
    if (wave == 3) {
        // mass of the slice above the range, in units of the range's top octave
        u128 ms = 0;
        if (ranged) {
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int t = kSB - 1 - 3 * lane - i;
                if (t >= 0 && (int)kBin0 + t > bt) {
                    const uint64_t w = bin_total(t);
                    if (w) ms += pack_mass(w, 127u + ((kBin0 + (uint32_t)t) >> 2) - exb_top);
                }
            }
        }
        const u128 tot = wave_sum(ms);
        if (lane == 0) { st[0] = (uint64_t)tot; st[1] = (uint64_t)(tot >> 64); }
    }
    // (the sub-bins are complete: the barrier above)
    if (wave == 0) {
        // Running counts and masses of the range from its top.  Lane l owns sub-bins 127 - 2l and 126 - 2l; a
        // sub-bin lies in one octave, ex octaves below the range's top.
        uint64_t w0 = 0, w1 = 0;
#pragma unroll
        for (int c = 0; c < kW1Rep; ++c) { w0 += s.sub[(127 - 2 * lane) * kW1Rep + c]; w1 += s.sub[(126 - 2 * lane) * kW1Rep + c]; }
        const uint32_t ex0 = (lo_bits + ((uint32_t)(127 - 2 * lane) << sh)) >> 23, ex1 = (lo_bits + ((uint32_t)(126 - 2 * lane) << sh)) >> 23;
        const uint32_t c0 = pack_count(w0), c1 = pack_count(w1);
        const u128 m0 = w0 ? pack_mass(w0, 127u + ex0 - exb_top) : (u128)0, m1 = w1 ? pack_mass(w1, 127u + ex1 - exb_top) : (u128)0;
        const uint32_t ci = wave_inclusive_scan(c0 + c1);
        const u128 mi = wave_inclusive_scan(m0 + m1);
        const uint32_t cc_hi = ci - c1, cc_lo = ci;
        const u128 mm_hi = mi - m1, mm_lo = mi;
        uint32_t *cum = v.cum + ((size_t)row * G + part) * kSB;
        s.cpc[127 - 2 * lane] = cc_hi; s.cpc[126 - 2 * lane] = cc_lo;
        cum[127 - 2 * lane] = cc_hi; cum[126 - 2 * lane] = cc_lo;
        st[2 + 2 * (127 - 2 * lane)] = (uint64_t)mm_hi; st[2 + 2 * (127 - 2 * lane) + 1] = (uint64_t)(mm_hi >> 64);
        st[2 + 2 * (126 - 2 * lane)] = (uint64_t)mm_lo; st[2 + 2 * (126 - 2 * lane) + 1] = (uint64_t)(mm_lo >> 64);
        if (lane == 0) { s.cpc[128] = 0; s.cpc[129] = 0; cum[128] = 0; st[2 + 256] = 0; st[2 + 257] = 0; }
        // The window: what the sample asked for, as far as it fits; else the widest stretch around the
        // expected threshold that does (lane l tries half-widths l and l + 64).
        const int wl0 = (int)gs.j_lo, wh0 = (int)gs.j_hi, je = (int)gs.j_est;
        auto inside = [&](int w) {
            const int lo = max(wl0, je - w), hi = min(wh0, je + w);
            return s.cpc[lo] - s.cpc[hi + 1];
        };
        const uint64_t fit0 = __ballot(inside(lane) <= (uint32_t)kW1Cap), fit1 = __ballot(inside(lane + 64) <= (uint32_t)kW1Cap);
        const int nfit = __popcll(fit0) + __popcll(fit1);       // counts grow with the width: the fitting widths are a prefix
        uint32_t wl = 1u, wh = 0u, wn = 0u;
        if (ranged && nfit != 0) {
            const int w = nfit - 1;
            wl = (uint32_t)max(wl0, je - w); wh = (uint32_t)min(wh0, je + w);
            wn = inside(w);
        }
        // where each sub-bin of the window begins among the tokens set aside (largest values first)
        const uint32_t top = s.cpc[min(wh, 127u) + 1];
        s.off[127 - 2 * lane] = s.cpc[128 - 2 * lane] - top;
        s.off[126 - 2 * lane] = cc_hi - top;
        if (lane == 0) {
            s.win_lo = wl; s.win_hi = wh; s.n = wn;
            PartHdr ph;
            ph.mkey = k; ph.cov = ranged ? (wl | wh << 8 | kWideValid) : 0u; ph.n = wn; ph.cut = 0u;
            v.hdr[(size_t)row * G + part] = ph;
        }
    }
    __syncthreads();                                     // the bins have been read: their memory becomes the staging area
    const uint32_t win_lo = s.win_lo, win_hi = s.win_hi, n = s.n;
    if (n != 0u) {
        const uint32_t rel = (127u - exb_top) << 23;     // bit patterns as if the range's top octave were [1, 2)
        // the window as bit patterns: one comparison per token
        const uint32_t w_lo = max(lo_bits + (win_lo << sh), lo_live), w_width = lo_bits + ((win_hi + 1u) << sh) - w_lo;
#pragma unroll
        for (int j = 0; j < R; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t b = eb[j * 4 + q];
                if (b - w_lo < w_width) {
                    const uint32_t slot = atomicAdd(&s.off[(b - lo_bits) >> sh], 1u);
                    if (slot < (uint32_t)kW1Cap) s.stage[slot] = ((uint64_t)(b + rel) << 32) | ((base4 + (uint32_t)j * NT) * 4u + (uint32_t)q);
                }
            }
    }
    __syncthreads();
    for (uint32_t i = (uint32_t)tid; i < min(n, (uint32_t)kW1Cap); i += NT) st[kW1Head + i] = s.stage[i];
}

template <int SLICE_LOG2>
__device__ __forceinline__ void wide1_finish_row(const Params &p, const StreamView &v, Lds &s, LdsB &t, const uint32_t row)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = v.G;
    const PartHdr *hdrs = v.hdr + (size_t)row * G;
    RowCtl *rc = p.ctl_end - 1 - row;

    if (tid == 0) { s.abort = 0; s.host_words = p.host_words; t.fail = 0; t.result = 0u; }
    PartHdr ph;
    ph.mkey = 0; ph.cov = 0; ph.n = 0; ph.cut = 0;
    if ((uint32_t)tid < G) ph = hdrs[tid];
    const uint64_t h0 = rc->rowhist[tid], h1 = rc->rowhist[tid + kThreads];
    rc->rowhist[tid] = 0; rc->rowhist[tid + kThreads] = 0;          // left clean for the next call
    const WideGuess gs = *reinterpret_cast<const WideGuess *>(rc->A);
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
    uint32_t kmax, kmin;
    {
        const uint32_t a = wave_max_u32(ph.mkey), b = wave_max_u32((uint32_t)tid < G ? ~ph.mkey : 0u);
        if (lane == 0) { s.u32[wave] = a; s.u32[kWaves + wave] = b; }
        __syncthreads();                                 // (everyone holds the guess: its words can go back to zero)
        kmax = s.u32[0]; kmin = s.u32[kWaves];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) { kmax = max(kmax, s.u32[w]); kmin = max(kmin, s.u32[kWaves + w]); }
        kmin = ~kmin;
    }
    if (tid < (int)(sizeof(WideGuess) / sizeof(uint64_t))) rc->A[tid] = 0;
    const float xmax = fkey_inv(kmax);
    const float M = __builtin_floorf(xmax);
    const bool mixed = !(M - __builtin_floorf(fkey_inv(kmin)) < 88.0f);
    if ((uint32_t)tid < G) {
        const float Mg = __builtin_floorf(fkey_inv(ph.mkey));
        const float d = M - Mg;
        t.delta[tid] = d >= 64.0f ? 64u : (uint32_t)d;
        t.m4[tid] = (uint32_t)(int)(Mg - 128.0f * __builtin_floorf(Mg * 0.0078125f)) * 4u;
    }
    for (int b = tid; b < (int)kBin0; b += kThreads) s.g[b] = 0;
    __syncthreads();
    level1_to_row_frame(s, v, row, M, mixed, h0, h1, t.delta, t.m4);
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
    const uint64_t top_k = (uint64_t)p.top_k;
    Found f = hist_find_level1<false>(s, top_k, p.top_p, lane, wave);
    const u128 D = s.D, P = s.P;
    const uint64_t rand64 = p.inj_u ? 0ull : t.rand64;
    auto slow = [&]() {
        finish_row_slow(p, s, t, row, xmax, rand64);
        if (tid == 0) {
            const uint32_t c = __hip_atomic_fetch_add(&p.hdr->n_need, 1u, __ATOMIC_RELAXED, RS_AGENT);
            if (c == 0u && p.host_words)                 // the call's first such row tells the caller's policy at once
                __hip_atomic_store(p.host_words + p.report, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    };

    // one tie of all the row's tokens: as on the streaming path
    if (f.cnt_bin == (uint32_t)p.V && bin_is_one_tie(s.g[f.bin], f.bin, e_bits_of(xmax, M))) {
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

    // The range in the row's frame, which must hold the level-1 boundary.  (The sample's frame is never
    // above the row's.)
    if (gs.state != 1u) return slow();
    const int bt = range_top_in_frame(gs.bin_top, gs.M, M);
    const int nb = 1 << gs.n_log2, lo_bin = bt + 1 - nb;
    if (bt > (int)kTop1 || (int)f.bin > bt || (int)f.bin < lo_bin) return slow();
    const uint32_t sh = 14u + gs.n_log2;
    const uint32_t shr = 127u - ((uint32_t)bt >> 2);                // octaves from the range's top octave up to [1, 2)
    // what the row holds above the range and in it, from the level-1 histogram
    uint32_t c_ab = 0, c_in = 0;
    u128 m_ab = 0;
    if (tid < kSB) {
        const int bin = (int)kBin0 + tid;
        const uint64_t w = s.g[bin];
        if (bin > bt) { c_ab = pack_count(w); if (w) m_ab = pack_mass(w, (uint32_t)bin >> 2); }
        else if (bin >= lo_bin) c_in = pack_count(w);
    }
    const uint32_t cnt_ar = block_sum_u32(s, c_ab, lane, wave);
    const uint32_t cnt_in = block_sum_u32(s, c_in, lane, wave);
    const u128 mass_ar = block_sum_u128(s, m_ab, lane, wave);
    // The row's running sums at the sub-bin edges: the slices' added up (edge 128 is zero by definition).
    // Every thread takes one edge and half of the slices, sixteen slices' loads in flight at a time; what a
    // slice that said nothing left behind is not added.
    if ((uint32_t)tid < G) t.take[tid] = ph.cov & kWideValid;
    __syncthreads();
    uint32_t Rc = 0;
    u128 Rm = 0;
    {
        const uint32_t edge = (uint32_t)tid & 127u, upper = (uint32_t)tid >> 7;
        const uint32_t g_mid = (G + 1u) >> 1, g_lo = upper ? g_mid : 0u, g_hi = upper ? G : g_mid;
        const uint32_t *cp0 = v.cum + (size_t)row * G * kSB + edge;
        const uint64_t *mp0 = v.stash + (size_t)row * G * kStashCap + 2 + 2 * edge;
        for (uint32_t g0 = g_lo; g0 < g_hi; g0 += 16u) {
            uint32_t c[16];
            uint64_t m0[16], m1[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const size_t g = min(g0 + (uint32_t)u, G - 1u);
                c[u] = cp0[g * kSB]; m0[u] = mp0[g * kStashCap]; m1[u] = mp0[g * kStashCap + 1];
            }
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (g0 + (uint32_t)u < g_hi && t.take[g0 + (uint32_t)u]) { Rc += c[u]; Rm += (u128)m0[u] | ((u128)m1[u] << 64); }
        }
        if (upper) { t.blo[edge] = (uint64_t)Rm; t.bhi[edge] = (uint64_t)(Rm >> 64); t.m4[edge] = Rc; }
    }
    __syncthreads();
    uint64_t *Rlo = s.cand, *Rhi = s.cand + 256, *Rcn = s.cand + 512;
    if (tid < 128) {
        Rm += (u128)t.blo[tid] | ((u128)t.bhi[tid] << 64);
        Rc += t.m4[tid];
        Rlo[tid] = (uint64_t)Rm; Rhi[tid] = (uint64_t)(Rm >> 64); Rcn[tid] = Rc;
    } else {
        Rc = 0; Rm = 0;
        if (tid == 128) { Rlo[128] = 0; Rhi[128] = 0; Rcn[128] = 0; }
    }
    const bool suff = tid < 129 && ((uint64_t)cnt_ar + Rc >= top_k || mass_ar + (Rm >> shr) >= P);
    {
        const uint64_t vote = __ballot(suff);
        __syncthreads();
        if (lane == 0) s.u32[wave] = vote ? (uint32_t)(wave * kWave + 64 - __builtin_clzll(vote)) : 0u;       // highest sufficient edge + 1
        __syncthreads();
    }
    uint32_t jb1 = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) jb1 = max(jb1, s.u32[w]);
    // Nothing of the range suffices, or what lies above it does already: the threshold is not in the range.
    // Counts that do not add up: some slice said nothing.  (Where the range reaches below 2^-40 of the
    // row's frame its lowest sub-bins hold dead tokens, which the slices counted in their own frames and
    // the row's histogram did not; the cut lies on a sub-bin edge.)
    const uint32_t lo_row = (uint32_t)lo_bin << 21;
    const uint32_t j_cut = lo_row < kEMinBits ? (kEMinBits - lo_row) >> sh : 0u;
    if (jb1 == 0u || jb1 == 129u || (uint32_t)Rcn[min(j_cut, 128u)] != cnt_in) return slow();
    const uint32_t jb = jb1 - 1u;
    {
        const u128 m_hi = (u128)Rlo[jb + 1] | ((u128)Rhi[jb + 1] << 64);
        f.cnt_above = cnt_ar + (uint32_t)Rcn[jb + 1];
        f.cnt_bin = (uint32_t)Rcn[jb] - (uint32_t)Rcn[jb + 1];
        f.mass_above = mass_ar + (m_hi >> shr);
    }

    // what every slice has of that sub-bin, and whether the window it set aside covers it
    uint32_t mine = 0, offs = 0;
    u128 kept_g = 0;                                     // kept weight of slice tid, so far without its listed tokens
    bool bad = false;
    if ((uint32_t)tid < G && (ph.cov & kWideValid)) {
        const uint64_t *st = v.stash + ((size_t)row * G + tid) * kStashCap;
        const uint32_t *cum = v.cum + ((size_t)row * G + tid) * kSB;
        const uint32_t wl = ph.cov & 255u, wh = (ph.cov >> 8) & 255u;
        const uint32_t c_hi = cum[jb + 1], c_lo = cum[jb];
        mine = c_lo - c_hi;
        if (mine) {
            if (jb < wl || jb > wh) bad = true;
            else offs = c_hi - cum[wh + 1];
        }
        const u128 a1 = (u128)st[0] | ((u128)st[1] << 64);
        const u128 m_hi = (u128)st[2 + 2 * (jb + 1)] | ((u128)st[2 + 2 * (jb + 1) + 1] << 64);
        kept_g = (a1 + m_hi) >> shr;
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

    // gather: entry i belongs to the first slice whose inclusive prefix exceeds i; a thread takes a run.
    // The bit patterns come relative to the range's top octave and go into the row's frame.
    {
        const uint64_t down = (uint64_t)(shr << 23) << 32;
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
                t.list[i] = v.stash[((size_t)row * G + g) * kStashCap + kW1Head + t.m4[g] + (i - gbase)] - down;
            }
        }
    }
    __syncthreads();

    // the remaining bits of the threshold, on the listed tokens (all of them lie in the sub-bin)
    uint32_t lo = ((uint32_t)lo_bin << 21) + (jb << sh), span = (1u << sh) - 1u;
    const uint32_t exb = lo >> 23;
    for (uint32_t lv = sh == 14u ? 3u : 2u; lv <= (uint32_t)kLevels && f.cnt_bin > 1u; ++lv) {
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
        const Target tg = tie_and_target(p, row, rand64, xmax, D, P, thr, f.cnt_above, f.cnt_bin, f.mass_above, kW1Rounds, true);
        s.bc64[1] = tg.w_tie; s.bc128[0] = tg.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    const u128 r = s.bc128[0];
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
__global__ void __launch_bounds__(kThreads) wide1_finish_kernel(const Params p, const StreamView v)
{
    __shared__ Lds s;
    __shared__ LdsB t;
    extern __shared__ __align__(16) unsigned char finish_dyn[];
    t.list = reinterpret_cast<uint64_t *>(finish_dyn);
    wide1_finish_row<SLICE_LOG2>(p, v, s, t, blockIdx.x);
}

}  // namespace rs
