// The cluster path: a row is worked by a cluster of workgroups that keep their slices in
// registers and exchange histograms, boundary tokens and kept masses through the row's record.
#pragma once

#include "rs_common.h"

namespace rs {

// What a workgroup keeps of its slice of a row from the first load to the end of the call.
template <int R, bool PEN>
struct Slice {
    uint32_t    eb[R * 4];       // l, then x, then bits(e), of this thread's 4R tokens
    float4      pen[PEN ? R : 1];
    RowCtl     *rc;
    const char *lrow;
    float4     *pn4;
    uint32_t    row, part, G;
    uint32_t    base4;           // float4 slots of this thread: base4 + j*256, valid while < V4 (a prefix of j)
    int         nv;              // how many of them are inside the row
    uint32_t    kmax_row;        // fkey(max x): of the slice at first, of the row once it is known
    uint32_t    h_used;          // cluster histograms this row has used and not yet cleared (bit i: rc->h[i])
    bool        mx_posted;       // my slot of the slice maxima is still to be cleared
};

template <int R, bool PEN>
__device__ __forceinline__ void slice_setup(const Params &p, Slice<R, PEN> &sl, uint32_t row, uint32_t part, uint32_t G)
{
    const uint32_t V4 = (uint32_t)p.V >> 2;
    sl.row = row; sl.part = part; sl.G = G;
    sl.rc = p.ctl_end - 1 - row;
    sl.base4 = part * (uint32_t)(kThreads * R) + (uint32_t)threadIdx.x;
    sl.nv = sl.base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - sl.base4 + kThreads - 1) / kThreads);
    sl.lrow = logits_row(p, row);
    sl.pn4 = PEN ? reinterpret_cast<float4 *>(p.penalties + (int64_t)row * p.V) : nullptr;
    sl.h_used = 0u; sl.mx_posted = false; sl.kmax_row = 0u;
}

// This call's 64 random bits of a row, into s.bc64[5] (one thread; the state is advanced once, at
// the end, by the row's first workgroup).
__device__ __forceinline__ void draw_rand(const Params &p, Lds &s, uint32_t row)
{
    if (threadIdx.x == 64 && !p.inj_u) {
        const uint32_t *st = p.rng + (size_t)row * 16;
        uint32_t o[4];
        philox4x32_10(st[2], st[3], st[4], st[5], st[0], st[1], o);
        s.bc64[5] = ((uint64_t)o[0] << 32) | o[1];
    }
}

// Step 1: load the slice once, scale it; returns the largest x of this thread's tokens.
template <int R, bool PEN>
__device__ __forceinline__ float slice_load(const Params &p, Slice<R, PEN> &sl)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = sl.G, row = sl.row, part = sl.part, base4 = sl.base4;
    const int nv = sl.nv;
    RowCtl *rc = sl.rc;
    auto &eb = sl.eb;
    auto &pen = sl.pen;
    const char *lrow = sl.lrow;
    float4 *pn4 = sl.pn4;
    uint32_t &kmax_row = sl.kmax_row;
    uint32_t &h_used = sl.h_used;
    bool &mx_posted = sl.mx_posted;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    (void)lane; (void)wave; (void)row; (void)part; (void)base4; (void)nv; (void)rc; (void)eb; (void)pen; (void)lrow; (void)pn4;
    (void)kmax_row; (void)h_used; (void)mx_posted; (void)V4; (void)G;
    float lmax;
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
        lmax = -3.402823466e+38f;
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
    }
    return lmax;
}

// Steps 1b-2 of the cluster path: slice maximum, e in the slice's frame, the level-1 histogram
// summed over the cluster and brought into the row's frame (s.g the row's, s.hm this slice's),
// the tokens in the registers re-based to it.  Returns false when a bounded wait gave up.
template <int R, bool PEN>
__device__ __forceinline__ bool slice_level1(const Params &p, Lds &s, Slice<R, PEN> &sl, float lmax)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = sl.G, row = sl.row, part = sl.part, base4 = sl.base4;
    const int nv = sl.nv;
    RowCtl *rc = sl.rc;
    auto &eb = sl.eb;
    auto &pen = sl.pen;
    const char *lrow = sl.lrow;
    float4 *pn4 = sl.pn4;
    uint32_t &kmax_row = sl.kmax_row;
    uint32_t &h_used = sl.h_used;
    bool &mx_posted = sl.mx_posted;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    (void)lane; (void)wave; (void)row; (void)part; (void)base4; (void)nv; (void)rc; (void)eb; (void)pen; (void)lrow; (void)pn4;
    (void)kmax_row; (void)h_used; (void)mx_posted; (void)V4; (void)G;
    kmax_row = block_max_u32(s, fkey(lmax), lane, wave);            // of this slice, for now
    for (int b = tid; b < kNB * kRepC; b += kThreads) s.hr[b] = 0;
    // every workgroup posts its key (never 0 for a finite x) in its own slot
    if (G > 1 && tid == 0) a_store(&rc->mx[part], kmax_row);
    __syncthreads();
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
    h_used = G > 1 ? 1u : 0u;
    mx_posted = G > 1;                                   // my slot is still to be cleared
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
    return true;
}

// Steps 3-7: threshold, tie weight, pick, penalties, leaving.  s.g and s.hm hold the level-1
// histograms in the row's frame, the registers the tokens' e in that frame, s.bc64[5] the row's
// random bits.  Returns false when a bounded wait gave up (the error word is set; the workgroup
// must leave at once).
template <int R, bool PEN>
__device__ __forceinline__ bool slice_finish(const Params &p, Lds &s, Slice<R, PEN> &sl)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t G = sl.G, row = sl.row, part = sl.part, base4 = sl.base4;
    const int nv = sl.nv;
    RowCtl *rc = sl.rc;
    auto &eb = sl.eb;
    auto &pen = sl.pen;
    const char *lrow = sl.lrow;
    float4 *pn4 = sl.pn4;
    uint32_t &kmax_row = sl.kmax_row;
    uint32_t &h_used = sl.h_used;
    bool &mx_posted = sl.mx_posted;
    const uint32_t V4 = (uint32_t)p.V >> 2;
    (void)lane; (void)wave; (void)row; (void)part; (void)base4; (void)nv; (void)rc; (void)eb; (void)pen; (void)lrow; (void)pn4;
    (void)kmax_row; (void)h_used; (void)mx_posted; (void)V4; (void)G;
    auto clear_used = [&]() {
        for (uint32_t i = 0; i <= (uint32_t)kLevels; ++i)
            if (h_used >> i & 1u) zero_slice(rc->h[i], (i == 0u || i == (uint32_t)kLevels) ? (uint32_t)kNB : 128u, part, G);
        h_used = 0u;
        if (mx_posted && tid == 0) a_store(&rc->mx[part], 0u);
        mx_posted = false;
    };
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
                guard.tick(s, p.hdr, 3u);
                const uint32_t total = block_sum_u32(s, valid, lane, wave);
                if (total == ncand + G) break;
                if (s.abort) return false;
                if (tid == 0) { s.seen = total; s.want = ncand + G; }
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
                guard.tick(s, p.hdr, 4u);
                const uint32_t total = block_sum_u32(s, valid, lane, wave);
                if (total == G) break;
                if (s.abort) return false;
                if (tid == 0) { s.seen = total; s.want = G; }
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
            if (PEN && !p.defer_pen && G > 1) a_store(&rc->index_p1, (uint32_t)idx + 1u);
            if (PEN) s.bc32[7] = (uint32_t)idx;
        }
    }

    // ---- 7. penalties: decay and one-hot add, from registers ---------------
    if (PEN && !p.defer_pen) {
        __syncthreads();
        if (G > 1) {
            if (tid == 0) {
                const uint64_t t0 = wall_clock64();
                uint32_t spins = 0, v;
                while ((v = a_load(&rc->index_p1)) == 0u) {
                    if ((++spins & 1023u) == 0 && (uint64_t)wall_clock64() - t0 > spin_limit(p.hdr)) {
                        give_up(s, p.hdr, 5u);
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
            if (tid == 0) {
                a_store(&rc->done, 0u); a_store(&rc->cursor, 0u); a_store(&rc->index_p1, 0u);
                a_store(&rc->arrived, 0u); a_store(&rc->verdict, 0u);       // set by the one-launch path
            }
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

// One slice of one row, start to finish.  Returns false when a bounded wait
// gave up (the error word is set; the workgroup must leave at once).
template <int R, bool PEN>
__device__ __forceinline__ bool sample_slice(const Params &p, Lds &s, const uint32_t row, const uint32_t part)
{
    Slice<R, PEN> sl;
    slice_setup(p, sl, row, part, p.G);
    if (threadIdx.x == 0) { s.who = row << 16 | part; s.seen = 0; s.want = 0; }
    // the call's first thread reports on the streaming call before it, if there was one (report_begin)
    const bool reporter = blockIdx.x == 0 && threadIdx.x == 0 && p.host_words != nullptr;
    PrevCall prev;
    prev.slow_rows = 0; prev.meta = 0;
    if (reporter) prev = report_begin(p);
    draw_rand(p, s, row);
    const float lmax = slice_load(p, sl);
    if (reporter) report_end(p, prev, false);
    if (!slice_level1(p, s, sl, lmax)) return false;
    return slice_finish(p, s, sl);
}

// The workgroups of a row wait for EACH OTHER (every exchange is all-to-all within the row).  A launch
// that the device holds all at once (256 CUs x the workgroups per CU the launch bounds guarantee)
// uses the hardware's workgroup ids: every workgroup becomes resident whatever else runs, so every
// wait ends.  A larger launch hands out (row, slice) by tickets (take_ticket), so that logical ids
// follow the order in which workgroups actually start: the hardware binds workgroup b of a launch to
// XCD b mod 8 before it starts, each XCD draws from a counter of its own, and the ids it holds at any
// time are the lowest of its residue not yet finished -- so the earliest unfinished row has, on every
// XCD, its workgroups running or next to start, and finishes; then the next one.  A row puts an
// eighth of its workgroups (at most 8 of 64) on each XCD, far fewer than an XCD holds.  A device
// partitioned below 256 CUs, or shared with other long-running kernels, can starve a row -- the waits
// are bounded for that case and end in RS_ERR_DEVICE rather than a hang.
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
    // A launch that the device holds all at once needs no tickets: every workgroup is resident whatever
    // the order they start in, and a few hundred fetch-adds on one word, served one after the other,
    // would hold the last workgroups back by microseconds.
    constexpr uint32_t kResident = 256u * (uint32_t)min_waves<R, PEN>();
    if (threadIdx.x == 0) {
        s.abort = 0; s.host_words = p.host_words;
        uint32_t t = blockIdx.x;
        if (gridDim.x > kResident) t = take_ticket(p.hdr);
        s.bc32[0] = t;
    }
    __syncthreads();
    const uint32_t ticket = s.bc32[0];
    const uint32_t row = ticket / p.G;
    sample_slice<R, PEN>(p, s, row, ticket - row * p.G);
}

}  // namespace rs
