// The row kernel: one workgroup of 1024 threads per row, the whole row (up to 65536 tokens) in its
// registers, one launch, one read of the logits, no workspace, no waits, no other kernel.
//
// A row of up to 65536 tokens fits the registers of one compute unit (64 tokens per thread), and
// then everything the other paths exchange between workgroups or kernels stays inside one
// workgroup: the maximum, e, the level-1 histogram in LDS, the radix selection of the threshold
// level by level (level 2 on the registers, the deeper ones on a list of the boundary bin's tokens
// in LDS when they fit), tie weight and target, and the pick by sums and scans of the kept weights
// in index order.  Its time hardly depends on the kept set, only on the row: it is the time of the
// vector instructions of e and of three passes over the registers, 64 tokens per thread with four
// waves per SIMD (measured, launch included: 14-18 us for 8192 tokens, 26 for 32768, 33 for 50304,
// 42 for 65536); a call of B rows takes ceil(B / 256) such times.  For kept sets of thousands of
// tokens in calls of 64 rows and more that is less than the general kernel's exchanges or the wide
// paths' launches cost; small calls and small kept sets are better off elsewhere.  Same integers as
// every other path.
#pragma once

#include "rs_common.h"

namespace rs {

constexpr int      kRowT      = 1024;                    // threads of the row kernel
constexpr int      kRowW      = kRowT / kWave;
constexpr int      kRowR      = 16;                      // groups of four tokens per thread at most: rows of up to 65536 tokens
static_assert(kRowMaxV == kRowT * kRowR * 4, "the row kernel's registers hold kRowMaxV tokens");
constexpr uint32_t kRowListW  = 768u;                    // tokens of the boundary bin a wave can list for levels 3 and 4
constexpr uint32_t kRowList   = kRowListW * 12u;         // the row's boundary bin is listed when it holds no more than this (16 waves: room to spare for uneven shares)
constexpr uint32_t kRowRounds = 10u;                     // DiagRow::rounds of a row finished here

struct LdsRowS {                      // what the shared helpers work on
    u128     D, P;
    Found    found;
    u128     bc128[2];
    uint64_t g[kNB];                  // the row's level-1 bins
    uint64_t hm[128];                 // a deeper level's bins
    uint64_t bc64[2];
    uint32_t bc32[8];
};
static_assert(kRowW * kRowListW / 2 >= (uint32_t)kNB * 8u, "the lists lie where the copies of the level-1 bins were");
struct LdsRow {
    LdsRowS  s;
    uint64_t hr8[kRowW * kRowListW / 2];   // level 1 while it is counted: eight copies of each bin (the first kNB * 8
                                      // words); later the waves' lists of the boundary bin's tokens (all of it)
    uint64_t lev[128 * 4];            // a deeper level while it is counted: four copies
    u128     wq[kRowW];               // per wave: kept weight of its stretch of the row
    u128     wq4[kRowW][4];           // the same, a quarter of the wave's groups at a time
    uint32_t nolist;                  // a wave's share of the boundary bin did not fit its list
    uint32_t wu[kRowW];
    uint64_t rand64;
};

__device__ __forceinline__ uint32_t row_max_u32(LdsRow &L, uint32_t v, int lane, int wave)
{
    v = wave_max_u32(v);
    __syncthreads();
    if (lane == 0) L.wu[wave] = v;
    __syncthreads();
    uint32_t r = L.wu[0];
#pragma unroll
    for (int w = 1; w < kRowW; ++w) r = max(r, L.wu[w]);
    return r;
}

// Wave w holds the stretch of G = ceil(V / 4 / 16) groups of four tokens from group w * G on, lane l its
// groups w * G + j * 64 + l (j < R): a load instruction of a wave reads 1 KB in one piece, and index
// order is wave, then j, then lane, then token.
template <int DT, int R>              // the logits' type; groups per thread (R * 1024 >= V / 4)
__global__ void __launch_bounds__(kRowT) row_kernel(const Params p)
{
    constexpr int kRowR = R;
    __shared__ LdsRow L;
    LdsRowS &s = L.s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t row = blockIdx.x;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t G = (V4 + (uint32_t)kRowW - 1u) / (uint32_t)kRowW;
    const uint32_t g0 = (uint32_t)wave * G + (uint32_t)lane;               // this thread's first group
    const uint32_t g_end = min(((uint32_t)wave + 1u) * G, V4);             // end of the wave's stretch
    const char *lrow = logits_row(p, row);
    // the call's first thread reports on the streaming call before it, if there was one (report_begin)
    const bool reporter = blockIdx.x == 0 && tid == 0 && p.host_words != nullptr;
    PrevCall prev;
    prev.slow_rows = 0; prev.meta = 0;
    if (reporter) prev = report_begin(p);
    for (int i = tid; i < kNB * 8; i += kRowT) L.hr8[i] = 0;
    if (tid == 0) L.nolist = 0u;

    // token (g0 + j * 64) * 4 + q sits in register j * 4 + q; slots past the end of the stretch read the
    // row's last group again (harmless for the maximum and the probe) and are set aside before anything is counted
    uint32_t eb[kRowR * 4];                              // l, then x, then bits(e)
    if constexpr (DT == RS_DTYPE_F32) {
        const uint4 *lg = reinterpret_cast<const uint4 *>(lrow);
#pragma unroll
        for (int j = 0; j < kRowR; ++j) {
            const uint4 l = load_once(lg + min(g0 + (uint32_t)(j * kWave), V4 - 1u));
            eb[j * 4 + 0] = l.x; eb[j * 4 + 1] = l.y; eb[j * 4 + 2] = l.z; eb[j * 4 + 3] = l.w;
        }
    } else {
        const uint2 *lh = reinterpret_cast<const uint2 *>(lrow);
        uint2 h[kRowR];
#pragma unroll
        for (int j = 0; j < kRowR; ++j) h[j] = load_once(lh + min(g0 + (uint32_t)(j * kWave), V4 - 1u));
#pragma unroll
        for (int j = 0; j < kRowR; ++j) widen4(h[j], DT, &eb[j * 4]);
    }
    // the row's random number, drawn while the loads are in flight; the row is always finished here
    if (tid == kWave && !p.inj_u) {
        uint32_t *rng_st = p.rng + (size_t)row * 16;
        uint32_t rs[6], o[4];
#pragma unroll
        for (int i = 0; i < 6; ++i) rs[i] = rng_st[i];
        philox4x32_10(rs[2], rs[3], rs[4], rs[5], rs[0], rs[1], o);
        L.rand64 = ((uint64_t)o[0] << 32) | o[1];
        rng_st[2] = rs[2] + 1u;
        if (rs[2] + 1u == 0u) rng_st[3] = rs[3] + 1u;
    }
    // x = l * c unless a NaN or an infinity shows up (see stream_kernel)
    constexpr int kSpecial = 0x207;
    float probe = 0.0f;
    float lmax = -3.402823466e+38f;
#pragma unroll
    for (int j = 0; j < kRowR; ++j) {
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
        for (int j = 0; j < kRowR; ++j) {
            const float x0 = sf(__uint_as_float(eb[j * 4])), x1 = sf(__uint_as_float(eb[j * 4 + 1]));
            const float x2 = sf(__uint_as_float(eb[j * 4 + 2])), x3 = sf(__uint_as_float(eb[j * 4 + 3]));
            lmax = fmaxf(lmax, fmaxf(fmaxf(x0, x1), fmaxf(x2, x3)));
            eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
            eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
        }
    }
    if (reporter) report_end(p, prev, false);
    const uint32_t kmax = row_max_u32(L, fkey(lmax), lane, wave);
    const float xmax = fkey_inv(kmax);
    const float M = __builtin_floorf(xmax);

    // e (not clamped at 2^-40: what lies below is dead and lands in bins nobody looks at) and level 1
#pragma unroll
    for (int j = 0; j < kRowR; ++j) {
        if (g0 + (uint32_t)(j * kWave) < g_end) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t b = e_bits_raw(__uint_as_float(eb[j * 4 + q]), M);
                eb[j * 4 + q] = b;
                atomicAdd(reinterpret_cast<unsigned long long *>(&L.hr8[(b >> 21) * 8u + (uint32_t)(lane & 7)]),
                          (unsigned long long)(kPackOne | (b & 0x7FFFFFu)));
            }
        } else {
            eb[j * 4] = 0; eb[j * 4 + 1] = 0; eb[j * 4 + 2] = 0; eb[j * 4 + 3] = 0;
        }
    }
    if (p.e_bits) {
        // diagnostics: e of every token, dead tokens as 0
        uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
        auto live = [](uint32_t b) { return b < kEMinBits ? 0u : b; };
#pragma unroll
        for (int j = 0; j < kRowR; ++j)
            if (g0 + (uint32_t)(j * kWave) < g_end)
                dst[g0 + (uint32_t)(j * kWave)] = make_uint4(live(eb[j * 4]), live(eb[j * 4 + 1]), live(eb[j * 4 + 2]), live(eb[j * 4 + 3]));
    }
    __syncthreads();
    if (tid < kNB) {
        uint64_t w = 0;
        if (tid >= (int)kBin0) {
#pragma unroll
            for (int c = 0; c < 8; ++c) w += L.hr8[tid * 8 + c];
        }
        s.g[tid] = w;
    }
    __syncthreads();
    const uint64_t top_k = (uint64_t)p.top_k;
    Found f = hist_find_level1<false, false, LdsRowS>(s, top_k, p.top_p, lane, wave);
    const u128 D = s.D, P = s.P;
    const uint64_t rand64 = p.inj_u ? 0ull : L.rand64;

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

    // ---- the threshold: radix selection on the registers, 7 bits a level ----
    const uint32_t exb = f.bin >> 2;
    uint32_t lo = f.bin << 21, span = (1u << 21) - 1u;
    bool one_tie = false;
    if (f.cnt_bin > 1u && f.cnt_above == 0u) {
        // a boundary bin that is one tie of the row's largest token: no further level needed, and counting
        // it would queue its tokens up at one address
        const uint32_t emax = e_bits_of(xmax, M);
        one_tie = bin_is_one_tie(s.g[f.bin], f.bin, emax);
        if (one_tie) { lo = emax; span = 0u; }
    }
    // The tokens of the boundary bin are listed while level 2 counts them (where the bin's copies were: they
    // are done with), every wave its own in a list of its own -- no counter to share, no wait: the place is
    // the wave's running count plus the lane's rank among the wave's candidates of that instruction -- if
    // the bin holds few enough for every wave's share to fit; levels 3 and 4 then read the lists, a few
    // entries per thread, and not the registers again.  A wave whose share does not fit after all (a sorted
    // row: the whole bin in one stretch) says so, and the levels go on from the registers.
    uint32_t *list = reinterpret_cast<uint32_t *>(L.hr8) + (uint32_t)wave * kRowListW;
    const bool use_list = f.cnt_bin <= kRowList;
    bool have_list = false;
    uint32_t nlist = 0u;                                 // wave-uniform
    for (uint32_t lv = 2; lv <= (uint32_t)kLevels && !one_tie && f.cnt_bin > 1u; ++lv) {
        const uint32_t dsh = level_shift(lv);
        if (tid < 128 * 4) L.lev[tid] = 0;
        __syncthreads();
        // the mask is made opaque so that the 64 words to add are built here, level by level, and not
        // kept in 128 registers across the levels
        uint32_t fmask = 0x7FFFFFu;
        asm volatile("" : "+v"(fmask));
        if (use_list && lv == 2u) {                      // count and list
#pragma unroll
            for (int j = 0; j < kRowR; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t b = eb[j * 4 + q];
                    const bool in = b - lo <= span;
                    const uint64_t cand = __builtin_amdgcn_ballot_w64(in);
                    if (in) {
                        atomicAdd(reinterpret_cast<unsigned long long *>(&L.lev[((b >> dsh) & 127u) * 4u + (uint32_t)(lane & 3)]),
                                  (unsigned long long)(kPackOne | (b & fmask)));
                        const uint32_t at = nlist + __builtin_amdgcn_mbcnt_hi((uint32_t)(cand >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)cand, 0u));
                        if (at < kRowListW) list[at] = b;
                    }
                    nlist += (uint32_t)__builtin_popcountll(cand);
                }
            if (nlist > kRowListW && lane == 0) L.nolist = 1u;
        } else if (!have_list) {                         // count, from the registers
#pragma unroll
            for (int j = 0; j < kRowR; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t b = eb[j * 4 + q];
                    if (b - lo <= span)
                        atomicAdd(reinterpret_cast<unsigned long long *>(&L.lev[((b >> dsh) & 127u) * 4u + (uint32_t)(lane & 3)]),
                                  (unsigned long long)(kPackOne | (b & fmask)));
                }
        } else {
            for (uint32_t i = (uint32_t)lane; i < nlist; i += (uint32_t)kWave) {
                const uint32_t b = list[i];
                if (b - lo <= span)
                    atomicAdd(reinterpret_cast<unsigned long long *>(&L.lev[((b >> dsh) & 127u) * 4u + (uint32_t)(lane & 3)]),
                              (unsigned long long)(kPackOne | (b & fmask)));
            }
        }
        __syncthreads();
        if (lv == 2u) have_list = use_list && L.nolist == 0u;
        if (tid < 128) s.hm[tid] = L.lev[tid * 4] + L.lev[tid * 4 + 1] + L.lev[tid * 4 + 2] + L.lev[tid * 4 + 3];
        __syncthreads();
        f = hist_find128(s, s.hm, f.cnt_above, f.mass_above, top_k, exb, lane, wave);
        lo |= f.bin << dsh;
        span = (1u << dsh) - 1u;
    }
    if (span != 0u) {                                    // a single token left in the range: the threshold itself
        if (have_list) {
            for (uint32_t i = (uint32_t)lane; i < nlist; i += (uint32_t)kWave)
                if (list[i] - lo <= span) s.bc32[6] = list[i];
        } else {
#pragma unroll
            for (int j = 0; j < kRowR; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (eb[j * 4 + q] - lo <= span) s.bc32[6] = eb[j * 4 + q];
        }
        __syncthreads();
        lo = s.bc32[6];
    }
    const uint32_t thr = lo;
    if (tid == 0) {
        const Target tg = tie_and_target(p, row, rand64, xmax, D, P, thr, f.cnt_above, f.cnt_bin, f.mass_above, kRowRounds, true);
        s.bc64[1] = tg.w_tie; s.bc128[0] = tg.r;
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1];
    const u128 r = s.bc128[0];

    // ---- the pick: kept weights in index order.  Every wave sums its stretch, a quarter of its groups at a
    // time; the wave whose stretch holds the target then finds it alone, in one quarter. ----
    constexpr int qb[5] = {0, (kRowR + 3) / 4, (2 * kRowR + 3) / 4, (3 * kRowR + 3) / 4, kRowR};
    // few kept tokens (f.cnt_above of them and f.cnt_bin ties): groups of four without one are skipped a wave at a time
    // (fewer than one kept token per wave and group on average: where most groups hold one the test only costs)
    const bool sparse = (uint64_t)(f.cnt_above + f.cnt_bin) * 256u < (uint64_t)(uint32_t)p.V;
    // (here a tie counts with the full weight of the threshold, and what the ties of the thread have too
    // much, tie_less each, is taken off the sum: a select less per token)
    auto weight = [=](uint32_t b) -> uint64_t {
        const uint32_t x = b >= thr ? ((b & 0x7FFFFFu) | 0x800000u) : 0u;
        return (uint64_t)x << (((b >> 23) - 87u) & 63u);
    };
    const uint64_t tie_less = w_of_bits(thr) - w_tie;    // w_tie <= the weight of the threshold
    u128 wtot = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        u128 mine = 0;
        uint32_t ties = 0u;
#pragma unroll
        for (int j = qb[q]; j < qb[q + 1]; ++j) {
            if (sparse) {
                const uint32_t m4 = max(max(eb[j * 4], eb[j * 4 + 1]), max(eb[j * 4 + 2], eb[j * 4 + 3]));
                if (__builtin_amdgcn_ballot_w64(m4 >= thr) == 0ull) continue;
            }
            mine += (u128)weight(eb[j * 4]) + weight(eb[j * 4 + 1]) + weight(eb[j * 4 + 2]) + weight(eb[j * 4 + 3]);
            ties += (uint32_t)(eb[j * 4] == thr) + (uint32_t)(eb[j * 4 + 1] == thr) + (uint32_t)(eb[j * 4 + 2] == thr) + (uint32_t)(eb[j * 4 + 3] == thr);
            // four weights at a time: the running sum is made opaque, or all the weights are worked out first
            // (two registers each) and summed as a tree
            uint64_t lo64 = (uint64_t)mine, hi64 = (uint64_t)(mine >> 64);
            asm volatile("" : "+v"(lo64), "+v"(hi64));
            mine = ((u128)hi64 << 64) | lo64;
        }
        mine -= (u128)ties * tie_less;
        const u128 t = wave_sum(mine);
        if (lane == 0) L.wq4[wave][q] = t;
        wtot += t;
    }
    if (lane == 0) L.wq[wave] = wtot;
    __syncthreads();
    if (wave == 0) {                                     // 1 <= r <= the sum of all kept weights: one stretch holds it
        const u128 t = lane < kRowW ? L.wq[lane] : (u128)0;
        const u128 inc = wave_inclusive_scan(t);
        const u128 exc = inc - t;
        if (lane < kRowW && exc < r && r <= inc) { s.bc32[7] = (uint32_t)lane; s.bc128[1] = r - exc; }
    }
    __syncthreads();
    if (wave != (int)s.bc32[7]) return;
    u128 rl = s.bc128[1];                                // 1 <= rl <= the kept weight of this wave's stretch
    int qstar = 0;
    for (int q = 0; q < 3; ++q) { const u128 t = L.wq4[wave][q]; if (rl > t) { rl -= t; qstar = q + 1; } else break; }
    const int jlo = qb[qstar], jhi = qb[qstar + 1];
    // (The weights are worked out again, from copies of the bits the compiler cannot see through: kept from
    // the first time they would fill 128 registers.)
    auto weight2 = [=](uint32_t b) -> uint64_t {
        asm volatile("" : "+v"(b));
        return (b > thr) ? w_of_bits(b) : (b == thr ? w_tie : 0ull);
    };
    bool found = false;
#pragma unroll
    for (int j = 0; j < kRowR; ++j) {
        if (found || j < jlo || j >= jhi) continue;
        const u128 w0 = weight2(eb[j * 4]), w1 = weight2(eb[j * 4 + 1]), w2 = weight2(eb[j * 4 + 2]), w3 = weight2(eb[j * 4 + 3]);
        const u128 m4 = w0 + w1 + w2 + w3;
        const u128 inc = wave_inclusive_scan(m4);
        const u128 t = lane63(inc);
        if (rl > t && j < jhi - 1) { rl -= t; continue; }
        found = true;
        const u128 exc = inc - m4;
        if (exc < rl && rl <= inc) {                     // exactly one lane
            const u128 rr = rl - exc;                    // 1 <= rr <= m4
            const int kk = (rr <= w0) ? 0 : (rr <= w0 + w1) ? 1 : (rr <= w0 + w1 + w2) ? 2 : 3;
            const int32_t idx = (int32_t)((g0 + (uint32_t)(j * kWave)) * 4u + (uint32_t)kk);
            p.out[row] = idx;
            if (p.diag) p.diag[row].index = idx;
        }
    }
}

}  // namespace rs
