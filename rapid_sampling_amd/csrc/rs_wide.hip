// Instantiations and the launchers of the wide paths.
#include "rs_wide1.h"

#ifndef RS_WIDE_NT
#define RS_WIDE_NT 512
#endif

namespace rs {

// A probe tells the caller's policy itself how it went: rows whose kept sets would not have fitted the
// stashes set the report word as they are found (wide_finish_row); if there was none, this one thread,
// behind the finish in stream order, clears the word, which the host set to "pending" with the call.
__global__ void probe_done_kernel(const Params p)
{
    if (threadIdx.x == 0 && a_load(&p.hdr->n_need) == 0u)
        __hip_atomic_store(p.host_words + p.report, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

hipError_t launch_wide(int slice_r, int32_t dtype, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v)
{
    const dim3 sgrid(B * v.G), sblock(kThreads);
#define RS_WIDE_DT(Rv, Lv, DTv) do {                                                                    \
        hipLaunchKernelGGL((stream_kernel<Rv, kThreads, DTv, true>), sgrid, sblock, 0, st, p, v);      \
        hipLaunchKernelGGL(wide_plan_kernel, dim3(B), dim3(kThreads), 0, st, p, v);                    \
        hipLaunchKernelGGL((wide_kernel<(Rv * 256 / RS_WIDE_NT), RS_WIDE_NT, DTv>), sgrid, dim3(RS_WIDE_NT), 0, st, p, v);                        \
        hipLaunchKernelGGL((wide_finish_kernel<Lv>), dim3(B), dim3(kThreads), finish_lds_bytes, st, p, v); } while (0)
#define RS_WIDE(Rv, Lv) do {                                                        \
        if (dtype == RS_DTYPE_F32) RS_WIDE_DT(Rv, Lv, RS_DTYPE_F32);               \
        else if (dtype == RS_DTYPE_BF16) RS_WIDE_DT(Rv, Lv, RS_DTYPE_BF16);        \
        else RS_WIDE_DT(Rv, Lv, RS_DTYPE_F16); } while (0)
    if (slice_r == 4) RS_WIDE(4, 12);
    else if (slice_r == 8) RS_WIDE(8, 13);
    else RS_WIDE(kStreamLongR, kStreamLongLog2);
#undef RS_WIDE
#undef RS_WIDE_DT
    if (p.probe && p.host_words) hipLaunchKernelGGL(probe_done_kernel, dim3(1), dim3(kWave), 0, st, p);
    return hipGetLastError();
}

hipError_t launch_wide1(int slice_r, int32_t dtype, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v)
{
    const dim3 sgrid(B * v.G), sblock(kThreads);
    hipLaunchKernelGGL(wide_sample_kernel, dim3(B), dim3(kW1SampleT), 0, st, p, v);
#define RS_W1_DT(Rv, Lv, DTv) do {                                                                      \
        hipLaunchKernelGGL((wide1_kernel<Rv, DTv>), sgrid, sblock, 0, st, p, v);                        \
        hipLaunchKernelGGL((wide1_finish_kernel<Lv>), dim3(B), sblock, finish_lds_bytes, st, p, v); } while (0)
#define RS_W1(Rv, Lv) do {                                                          \
        if (dtype == RS_DTYPE_F32) RS_W1_DT(Rv, Lv, RS_DTYPE_F32);                 \
        else if (dtype == RS_DTYPE_BF16) RS_W1_DT(Rv, Lv, RS_DTYPE_BF16);          \
        else RS_W1_DT(Rv, Lv, RS_DTYPE_F16); } while (0)
    if (slice_r == 4) RS_W1(4, 12);
    else if (slice_r == 8) RS_W1(8, 13);
    else RS_W1(kStreamLongR, kStreamLongLog2);
#undef RS_W1
#undef RS_W1_DT
    return hipGetLastError();
}

}  // namespace rs
