// MI355X (gfx950) token sampler: kernels and the C ABI of include/rapid_sampling.h.
//
// One launch per call.  A row of V logits is worked by a CLUSTER of G
// workgroups of 256 threads; each thread keeps R float4 (4R tokens) of the row
// in registers for the whole call, so the row is read from HBM exactly once
// and every later pass runs out of the register file.  Workgroups of a
// cluster meet at device-scope barriers (an arrival counter per row in the
// workspace); everything they exchange is an integer sum, a max or a min, so
// the result does not depend on G, R or arrival order.
//
// Steps per row (reference lines in /root/reference/sampling.cu):
//   1  x = sf((sf(l) - pen) * c), row max            :208-227, :547-559
//   2  e = exp2(x - max) kept as bit patterns, D      :228-258
//   3  4-way threshold search on bit patterns         :261-329
//   4  smallest kept e, counts and mass above it      :332-355
//   5  tie weight                                     :365-371
//   6  inverse-CDF pick in index order                :374-426
//   7  penalty decay + one-hot add, in place          :427-437
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "rapid_sampling.h"
#include "rs_device.h"

namespace rs {

constexpr int      kThreads   = 256;          // 4 waves, one per SIMD
constexpr int      kWaves     = kThreads / kWave;
constexpr int      kMaxParts  = 256;          // workgroups per row, at most
constexpr int      kMaxRounds = 24;           // search passes, at most (range <= 2^30)
constexpr uint64_t kSpinLimit = 200000000ull; // 2 s of the 100 MHz wall clock

struct alignas(256) WsHeader {
    uint32_t ticket;      // next logical workgroup id of the running launch
    uint32_t finished;    // workgroups that have left the running launch
    int32_t  error;       // sticky RS_ERR_DEVICE
    uint32_t pad[61];
};

struct RoundSlot {
    uint32_t c[3];
    uint32_t pad;
    uint64_t m[3];
};

struct alignas(256) RowCtl {
    uint32_t arrive;      // barrier arrivals so far
    uint32_t done;        // workgroups finished with this row
    uint32_t maxkey;      // max of fkey(x)
    uint32_t emin_inv;    // max of ~bits(e)            -> emin
    uint32_t thr_inv;     // max of ~bits(e), e >= left -> smallest kept e
    uint32_t n_gt, n_eq;
    int32_t  index;
    uint64_t D, G;
    RoundSlot round[kMaxRounds];
    uint64_t W[kMaxParts];   // kept weight of each workgroup's slice
};

struct Params {
    const float *logits;
    float       *penalties;
    int32_t     *out;
    uint32_t    *rng;          // 16 words per row, or null
    const float *inj_u;        // or null
    rs_row_diag *diag;         // or null
    uint32_t    *e_bits;       // or null
    WsHeader    *hdr;
    RowCtl      *ctl;
    int64_t      row_stride;
    int32_t      B, V;
    uint32_t     G;            // workgroups per row
    float        presence, repetition, decay, c;
    int32_t      top_k;
    float        top_p;
};

#define RS_AGENT __HIP_MEMORY_SCOPE_AGENT

template <typename T> __device__ __forceinline__ T a_load(const T *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, RS_AGENT); }
template <typename T> __device__ __forceinline__ void a_store(T *p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, RS_AGENT); }
template <typename T> __device__ __forceinline__ void a_add(T *p, T v) { __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, RS_AGENT); }
template <typename T> __device__ __forceinline__ void a_max(T *p, T v) { __hip_atomic_fetch_max(p, v, __ATOMIC_RELAXED, RS_AGENT); }

// Hides a register from the optimiser for one use, so that work derived from
// the resident tokens (their fixed-point weights) is redone in each pass
// instead of being hoisted out of the loops and kept in two more registers
// per token.
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// Workgroup-local staging in LDS.
struct Lds {
    uint64_t u64[kWaves * 4];
    uint32_t u32[kWaves * 4];
    uint64_t bc64[8];       // broadcast slots
    uint32_t bc32[8];
    uint64_t wj[kWaves][32];
    uint64_t tj[32];
    int      abort;
};

// Sum of (c0,c1,c2 | m0,m1,m2) over the workgroup; result valid in thread 0.
__device__ __forceinline__ void block_sum3(Lds &s, uint32_t c[3], uint64_t m[3], int lane, int wave)
{
#pragma unroll
    for (int i = 0; i < 3; ++i) { c[i] = wave_sum(c[i]); m[i] = wave_sum(m[i]); }
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 3; ++i) { s.u32[wave * 4 + i] = c[i]; s.u64[wave * 4 + i] = m[i]; }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            uint32_t cc = 0; uint64_t mm = 0;
            for (int w = 0; w < kWaves; ++w) { cc += s.u32[w * 4 + i]; mm += s.u64[w * 4 + i]; }
            c[i] = cc; m[i] = mm;
        }
    }
}

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

__device__ __forceinline__ uint64_t block_sum_u64(Lds &s, uint64_t v, int lane, int wave)
{
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) s.u64[wave] = v;
    __syncthreads();
    uint64_t r = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) r += s.u64[w];
    return r;
}

// Meet the other workgroups of the row.  Thread 0 has issued this
// workgroup's contributions (relaxed device-scope atomics) before the call.
// Returns false when the wait gave up (sticky error set).
__device__ __forceinline__ bool cluster_barrier(Lds &s, RowCtl *rc, WsHeader *hdr, uint32_t target)
{
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(&rc->arrive, 1u, __ATOMIC_RELEASE, RS_AGENT);
        const uint64_t t0 = wall_clock64();
        uint32_t spins = 0;
        while (__hip_atomic_load(&rc->arrive, __ATOMIC_ACQUIRE, RS_AGENT) < target) {
            __builtin_amdgcn_s_sleep(1);
            if ((++spins & 255u) == 0 && wall_clock64() - t0 > kSpinLimit) {
                a_store(&hdr->error, (int32_t)RS_ERR_DEVICE);
                s.abort = 1;
                break;
            }
        }
    }
    __syncthreads();
    return s.abort == 0;
}

template <int R, bool PEN>
__global__ void __launch_bounds__(kThreads) sample_kernel(const Params p)
{
    __shared__ Lds s;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;

    if (tid == 0) {
        s.abort = 0;
        s.bc32[0] = __hip_atomic_fetch_add(&p.hdr->ticket, 1u, __ATOMIC_RELAXED, RS_AGENT);
    }
    __syncthreads();
    const uint32_t ticket = s.bc32[0];
    const uint32_t G = p.G;
    const uint32_t row = ticket / G, part = ticket - row * G;
    RowCtl *rc = p.ctl + row;
    uint32_t bar = 0;                                   // barriers passed

    const uint32_t V4 = (uint32_t)p.V >> 2;
    const uint32_t base4 = part * (uint32_t)(kThreads * R) + (uint32_t)tid;
    // float4 slots of this thread: base4 + j*256, valid while < V4 (a prefix of j)
    const int nv = base4 >= V4 ? 0 : (int)min((uint32_t)R, (V4 - base4 + kThreads - 1) / kThreads);

    const float4 *lg = reinterpret_cast<const float4 *>(p.logits + (int64_t)row * p.row_stride);
    float4 *pn4 = PEN ? reinterpret_cast<float4 *>(p.penalties + (int64_t)row * p.V) : nullptr;

    uint32_t eb[R * 4];                                 // x, then bits(e)
    float4 pen[PEN ? R : 1];

    // ---- 1. load once, scale, local max ---------------------------------
    {
        float4 l[R];
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t i4 = min(base4 + (uint32_t)(j * kThreads), V4 - 1);
            l[j] = lg[i4];
            if (PEN) pen[j] = pn4[i4];
        }
        float lmax = -3.402823466e+38f;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            float x0, x1, x2, x3;
            if (PEN) {
                x0 = sf((sf(l[j].x) - pen[j].x) * p.c);
                x1 = sf((sf(l[j].y) - pen[j].y) * p.c);
                x2 = sf((sf(l[j].z) - pen[j].z) * p.c);
                x3 = sf((sf(l[j].w) - pen[j].w) * p.c);
            } else {
                x0 = sf(l[j].x * p.c); x1 = sf(l[j].y * p.c);
                x2 = sf(l[j].z * p.c); x3 = sf(l[j].w * p.c);
            }
            if (j < nv) lmax = fmaxf(lmax, fmaxf(fmaxf(x0, x1), fmaxf(x2, x3)));
            eb[j * 4 + 0] = __float_as_uint(x0); eb[j * 4 + 1] = __float_as_uint(x1);
            eb[j * 4 + 2] = __float_as_uint(x2); eb[j * 4 + 3] = __float_as_uint(x3);
        }
        const uint32_t k = block_max_u32(s, fkey(lmax), lane, wave);
        if (tid == 0) a_max(&rc->maxkey, k);
    }
    if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
    if (tid == 0) s.bc32[1] = a_load(&rc->maxkey);
    __syncthreads();
    const float xmax = fkey_inv(s.bc32[1]);

    // ---- 2. e = exp2(x - max) in place, D, emin ---------------------------
    {
        uint64_t dl = 0;
        uint32_t einv = 0;
#pragma unroll
        for (int j = 0; j < R; ++j) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t b = __float_as_uint(exp2c(__uint_as_float(eb[j * 4 + k]) - xmax));
                eb[j * 4 + k] = b;
                if (j < nv) { dl += q_of_bits(b); einv = max(einv, ~b); }
            }
        }
        dl = block_sum_u64(s, dl, lane, wave);
        einv = block_max_u32(s, einv, lane, wave);
        if (tid == 0) { a_add(&rc->D, dl); a_max(&rc->emin_inv, einv); }
        if (p.e_bits) {
            uint4 *dst = reinterpret_cast<uint4 *>(p.e_bits + (int64_t)row * p.V);
#pragma unroll
            for (int j = 0; j < R; ++j)
                if (j < nv) dst[base4 + j * kThreads] = make_uint4(eb[j * 4], eb[j * 4 + 1], eb[j * 4 + 2], eb[j * 4 + 3]);
        }
    }
    if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
    if (tid == 0) { s.bc64[0] = a_load(&rc->D); s.bc32[2] = ~a_load(&rc->emin_inv); }
    __syncthreads();
    const uint64_t D = s.bc64[0];
    const uint32_t emin = s.bc32[2];
    const uint64_t P = ceil_mul(p.top_p, D);
    const uint64_t top_k = (uint64_t)p.top_k;

    // ---- 3. quaternary search on bit patterns ------------------------------
    // e_max is exp2c(0) = 1.0 exactly, so the upper end starts at bits(1.0)+1.
    uint32_t left = emin, right = 0x3F800000u + 1u;
    uint64_t cnt_x = (uint64_t)p.V, mass_x = D;
    uint32_t rounds = 0;
    while ((cnt_x > top_k || mass_x > P) && left < right - 1) {
        if (rounds >= (uint32_t)kMaxRounds) {            // cannot happen: the range shrinks 4x per pass
            if (tid == 0) a_store(&p.hdr->error, (int32_t)RS_ERR_DEVICE);
            return;
        }
        const uint32_t pz = (left + right) / 2;
        const uint32_t py = (left + pz) / 2;
        const uint32_t pw = (pz + right) / 2;
        uint32_t c[3] = {0, 0, 0};
        uint64_t m[3] = {0, 0, 0};
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j < nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t b = opaque(eb[j * 4 + k]);
                    const uint64_t q = q_of_bits(b);
                    if (b >= py) { c[0]++; m[0] += q; }
                    if (b >= pz) { c[1]++; m[1] += q; }
                    if (b >= pw) { c[2]++; m[2] += q; }
                }
            }
        }
        block_sum3(s, c, m, lane, wave);
        RoundSlot *slot = &rc->round[rounds];
        if (tid == 0) {
#pragma unroll
            for (int i = 0; i < 3; ++i) { a_add(&slot->c[i], c[i]); a_add(&slot->m[i], m[i]); }
        }
        if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
        if (tid == 0) {
#pragma unroll
            for (int i = 0; i < 3; ++i) { s.bc32[4 + i] = a_load(&slot->c[i]); s.bc64[4 + i] = a_load(&slot->m[i]); }
        }
        __syncthreads();
        const uint64_t cy = s.bc32[4], cz = s.bc32[5], cw = s.bc32[6];
        const uint64_t my = s.bc64[4], mz = s.bc64[5], mw = s.bc64[6];
        ++rounds;
        if (cy < top_k && my < P)      { right = py; }
        else if (cz < top_k && mz < P) { left = py; right = pz; cnt_x = cy; mass_x = my; }
        else if (cw < top_k && mw < P) { left = pz; right = pw; cnt_x = cz; mass_x = mz; }
        else                           { left = pw; cnt_x = cw; mass_x = mw; }
    }

    // ---- 4. smallest kept e, then counts and mass above it ------------------
    {
        uint32_t tinv = 0;
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) { const uint32_t b = eb[j * 4 + k]; if (b >= left) tinv = max(tinv, ~b); }
            }
        tinv = block_max_u32(s, tinv, lane, wave);
        if (tid == 0) a_max(&rc->thr_inv, tinv);
    }
    if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
    if (tid == 0) s.bc32[3] = ~a_load(&rc->thr_inv);
    __syncthreads();
    const uint32_t thr = s.bc32[3];
    {
        uint32_t c[3] = {0, 0, 0};
        uint64_t m[3] = {0, 0, 0};
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < nv) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t b = opaque(eb[j * 4 + k]);
                    if (b > thr) { c[0]++; m[0] += q_of_bits(b); }
                    if (b == thr) c[1]++;
                }
            }
        block_sum3(s, c, m, lane, wave);
        if (tid == 0) { a_add(&rc->n_gt, c[0]); a_add(&rc->n_eq, c[1]); a_add(&rc->G, m[0]); }
    }
    if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;

    // ---- 5. tie weight, total S, target r (every workgroup, identically) ----
    if (tid == 0) {
        const uint32_t n_gt = a_load(&rc->n_gt), n_eq = a_load(&rc->n_eq);
        const uint64_t Gm = a_load(&rc->G);
        const uint64_t q_thr = q_of_bits(thr);
        uint64_t w_tie = q_thr;
        const uint64_t a = (P > Gm) ? (P - Gm) / n_eq : 0;
        const uint64_t bk = ((uint32_t)p.top_k > n_gt) ? (q_thr * (uint64_t)((uint32_t)p.top_k - n_gt)) / n_eq : 0;
        if (a < w_tie) w_tie = a;
        if (bk < w_tie) w_tie = bk;
        if (w_tie == 0 && Gm == 0) w_tie = 1;
        const uint64_t S = Gm + (uint64_t)n_eq * w_tie;
        uint64_t r;
        if (p.inj_u) r = ceil_mul(p.inj_u[row], S);
        else {
            const uint32_t *st = p.rng + (size_t)row * 16;
            uint32_t o[4];
            philox4x32_10(st[2], st[3], st[4], st[5], st[0], st[1], o);
            r = r_from_bits(((uint64_t)o[0] << 32) | o[1], S);
        }
        s.bc64[1] = w_tie; s.bc64[2] = S; s.bc64[3] = r;
        if (p.diag && part == 0) {
            rs_row_diag *d = p.diag + row;
            d->xmax = xmax; d->emin_bits = emin; d->D = D; d->P = P;
            d->left_bits = left; d->thr_bits = thr; d->rounds = rounds;
            d->n_gt = n_gt; d->n_eq = n_eq; d->G = Gm; d->w_tie = w_tie; d->S = S; d->r = r;
        }
    }
    __syncthreads();
    const uint64_t w_tie = s.bc64[1], r = s.bc64[3];

    // ---- 6. inverse CDF: which workgroup, which float4 slot, which thread ---
    auto weight = [&](uint32_t b) -> uint64_t {
        b = opaque(b);
        return (b > thr) ? q_of_bits(b) : (b == thr ? w_tie : 0);
    };
    auto slot_weight = [&](int j) -> uint64_t {         // weight of float4 slot j of this thread
        return weight(eb[j * 4]) + weight(eb[j * 4 + 1]) + weight(eb[j * 4 + 2]) + weight(eb[j * 4 + 3]);
    };
    uint64_t wloc = 0;
#pragma unroll
    for (int j = 0; j < R; ++j)
        if (j < nv) wloc += slot_weight(j);
    const uint64_t wblock = block_sum_u64(s, wloc, lane, wave);
    if (tid == 0) a_store(&rc->W[part], wblock);
    if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
    uint64_t before = 0;
    for (uint32_t i = tid; i < part; i += kThreads) before += a_load(&rc->W[i]);
    before = block_sum_u64(s, before, lane, wave);
    const bool owner = before < r && r <= before + wblock;   // block-uniform

    if (owner) {
        uint64_t rl = r - before;                        // 1 <= rl <= wblock
        // totals per float4 slot j over the workgroup
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint64_t t = wave_sum(j < nv ? slot_weight(j) : 0ull);
            if (lane == 0) s.wj[wave][j] = t;
        }
        __syncthreads();
        if (tid < R) { uint64_t t = 0; for (int w = 0; w < kWaves; ++w) t += s.wj[w][tid]; s.tj[tid] = t; }
        __syncthreads();
        int jstar = 0;
        for (int j = 0; j < R - 1; ++j) { const uint64_t t = s.tj[j]; if (rl > t) { rl -= t; jstar = j + 1; } else break; }
        // rl <= wblock = sum of tj, so rl now lies inside slot jstar
        uint32_t e4[4] = {0, 0, 0, 0};
        bool have = false;
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j == jstar) { have = j < nv; e4[0] = eb[j * 4]; e4[1] = eb[j * 4 + 1]; e4[2] = eb[j * 4 + 2]; e4[3] = eb[j * 4 + 3]; }
        const uint64_t w0 = have ? weight(e4[0]) : 0, w1 = have ? weight(e4[1]) : 0;
        const uint64_t w2 = have ? weight(e4[2]) : 0, w3 = have ? weight(e4[3]) : 0;
        const uint64_t mine = w0 + w1 + w2 + w3;
        // inclusive scan over the 256 threads of slot jstar
        uint64_t inc = wave_inclusive_scan_u64(mine, lane);
        __syncthreads();
        if (lane == kWave - 1) s.u64[wave] = inc;
        __syncthreads();
        uint64_t woff = 0;
        for (int w = 0; w < wave; ++w) woff += s.u64[w];
        inc += woff;
        const uint64_t exc = inc - mine;
        if (exc < rl && rl <= inc) {                      // exactly one thread
            const uint64_t rr = rl - exc;                 // 1 <= rr <= mine
            const int kk = (rr <= w0) ? 0 : (rr <= w0 + w1) ? 1 : (rr <= w0 + w1 + w2) ? 2 : 3;
            const int32_t idx = (int32_t)((base4 + (uint32_t)jstar * kThreads) * 4 + (uint32_t)kk);
            p.out[row] = idx;
            if (p.diag) p.diag[row].index = idx;
            if (PEN) a_store(&rc->index, idx);
        }
    }

    // ---- 7. penalties: decay and one-hot add, from registers ---------------
    if (PEN) {
        if (!cluster_barrier(s, rc, p.hdr, ++bar * G)) return;
        if (tid == 0) s.bc32[7] = (uint32_t)a_load(&rc->index);
        __syncthreads();
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
    if (tid == 0) {
        if (part == 0 && !p.inj_u) {
            uint32_t *st = p.rng + (size_t)row * 16;
            const uint32_t lo = st[2] + 1;
            st[2] = lo;
            if (lo == 0) st[3] += 1;
        }
        s.bc32[0] = __hip_atomic_fetch_add(&rc->done, 1u, __ATOMIC_ACQ_REL, RS_AGENT);
    }
    __syncthreads();
    if (s.bc32[0] == G - 1) {
        // last workgroup out of this row: nobody reads the record any more
        uint32_t *w = reinterpret_cast<uint32_t *>(rc);
        for (uint32_t i = tid; i < sizeof(RowCtl) / 4; i += kThreads) a_store(&w[i], 0u);
    }
    __syncthreads();
    if (tid == 0) {
        const uint32_t f = __hip_atomic_fetch_add(&p.hdr->finished, 1u, __ATOMIC_ACQ_REL, RS_AGENT);
        if (f == gridDim.x - 1) { a_store(&p.hdr->finished, 0u); a_store(&p.hdr->ticket, 0u); }
    }
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

// ------------------------------------------------------------ host side ----

struct Geometry { int R; uint32_t G; };

// Tokens per thread (4R) and workgroups per row.  Large batches take long
// slices (few barriers' worth of peers, deep loads); a lone row is cut into
// ~64 slices so that many CUs pull it from HBM at once.
static Geometry choose_geometry(int32_t B, int32_t V, bool pen)
{
    const uint32_t V4 = (uint32_t)V / 4;
    const int maxR = pen ? 16 : 32;
    const char *force = getenv("RS_FORCE_R");
    auto parts = [&](int R) { return (V4 + (uint32_t)(kThreads * R) - 1) / (uint32_t)(kThreads * R); };
    if (force) {
        int R = atoi(force);
        if ((R == 1 || R == 2 || R == 4 || R == 8 || R == 16 || R == 32) && R <= maxR && parts(R) <= (uint32_t)kMaxParts)
            return {R, parts(R)};
    }
    const uint64_t want[2] = {512, 64};
    for (uint64_t w : want)
        for (int R = maxR; R >= 1; R /= 2)
            if (parts(R) <= (uint32_t)kMaxParts && (uint64_t)B * parts(R) >= w) return {R, parts(R)};
    for (int R = 1; R <= maxR; R *= 2)
        if (parts(R) <= (uint32_t)kMaxParts) return {R, parts(R)};
    return {maxR, parts(maxR)};
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

}  // namespace rs

using namespace rs;

extern "C" {

int rs_version(void) { return 100; }

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
    *bytes = sizeof(WsHeader) + (size_t)B * sizeof(RowCtl);
    return RS_OK;
}

int rs_workspace_init(void *ws, size_t bytes, void *stream)
{
    if (!ws) return RS_ERR_NULL;
    if (bytes < sizeof(WsHeader) || ((uintptr_t)ws & 255)) return RS_ERR_WORKSPACE;
    return hipMemsetAsync(ws, 0, bytes, (hipStream_t)stream) == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
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
    if (!logits || !out || !workspace || (!rng_state && !injected_u)) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    if (!(top_k >= 1 && top_k <= V) || !(top_p > 0.0f && top_p <= 1.0f) || !(log2e_inv_temp > 0.0f)) return RS_ERR_ARG;
    if (((uintptr_t)logits & 15) || (B > 1 && (row_stride & 3)) || ((uintptr_t)penalties & 15) || ((uintptr_t)e_bits & 15))
        return RS_ERR_ALIGN;
    size_t need = 0;
    rs_workspace_bytes(B, V, &need);
    if (workspace_bytes < need || ((uintptr_t)workspace & 255)) return RS_ERR_WORKSPACE;

    const bool pen = penalties != nullptr;
    const Geometry g = choose_geometry(B, V, pen);
    Params p;
    p.logits = logits; p.penalties = penalties; p.out = out;
    p.rng = (uint32_t *)rng_state; p.inj_u = injected_u; p.diag = diag; p.e_bits = e_bits;
    p.hdr = (WsHeader *)workspace;
    p.ctl = (RowCtl *)((char *)workspace + sizeof(WsHeader));
    p.row_stride = row_stride; p.B = B; p.V = V; p.G = g.G;
    p.presence = presence; p.repetition = repetition; p.decay = decay; p.c = log2e_inv_temp;
    p.top_k = top_k; p.top_p = top_p;
    const dim3 grid((uint32_t)B * g.G);
    const hipError_t e = pen ? launch_sample<true>(g.R, grid, (hipStream_t)stream, p)
                             : launch_sample<false>(g.R, grid, (hipStream_t)stream, p);
    return e == hipSuccess ? RS_OK : RS_ERR_LAUNCH;
}

int rs_floor_read(const float *logits, int64_t row_stride, int32_t *out, int32_t B, int32_t V, void *stream)
{
    if (!logits || !out) return RS_ERR_NULL;
    if (!(V > 0 && V <= 1048576 && V % 4 == 0)) return RS_ERR_VOCAB;
    if (B <= 0) return RS_ERR_BATCH;
    const Geometry g = choose_geometry(B, V, false);
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
