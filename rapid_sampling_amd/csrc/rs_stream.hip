// Instantiations and launchers of the streaming kernels.
#include "rs_stream.h"

namespace rs {

constexpr int kStreamNT = 256;

hipError_t launch_stream(int slice_r, int32_t dtype, bool keep, uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p,
                         const StreamView &v)
{
    const dim3 sgrid(B * v.G);
    // keep: the call keeps every live token; its kernels neither fill nor read stashes, and the finish needs no list.
    // NTv threads with Rv groups of four tokens each: a slice of 4 Rv NTv tokens
#ifndef RS_LONG_NT
#define RS_LONG_NT 256
#endif
#define RS_STREAM(Rv, NTv, Lv, KEEPv) do {                                                                                         \
        if (dtype == RS_DTYPE_F32) hipLaunchKernelGGL((stream_kernel<Rv, NTv, RS_DTYPE_F32, KEEPv>), sgrid, dim3(NTv), 0, st, p, v);       \
        else if (dtype == RS_DTYPE_BF16) hipLaunchKernelGGL((stream_kernel<Rv, NTv, RS_DTYPE_BF16, KEEPv>), sgrid, dim3(NTv), 0, st, p, v); \
        else hipLaunchKernelGGL((stream_kernel<Rv, NTv, RS_DTYPE_F16, KEEPv>), sgrid, dim3(NTv), 0, st, p, v);                             \
        hipLaunchKernelGGL((finish_kernel<Lv, KEEPv>), dim3(B), dim3(kThreads), KEEPv ? 0 : finish_lds_bytes, st, p, v); } while (0)
    if (slice_r == 4) { if (keep) RS_STREAM(4, 256, 12, true); else RS_STREAM(4, 256, 12, false); }
    else if (slice_r == 8) { if (keep) RS_STREAM(8, 256, 13, true); else RS_STREAM(8, 256, 13, false); }
    else { if (keep) RS_STREAM((kStreamLongR * 256 / RS_LONG_NT), RS_LONG_NT, kStreamLongLog2, true); else RS_STREAM((kStreamLongR * 256 / RS_LONG_NT), RS_LONG_NT, kStreamLongLog2, false); }
#undef RS_STREAM
    return hipGetLastError();
}

hipError_t launch_stream_pen(uint32_t B, size_t finish_lds_bytes, hipStream_t st, const Params &p, const StreamView &v)
{
    hipLaunchKernelGGL((stream_pen_kernel<kStreamLongR>), dim3(B * v.G), dim3(kThreads), 0, st, p, v);
    hipLaunchKernelGGL((finish_kernel<kStreamLongLog2>), dim3(B), dim3(kThreads), finish_lds_bytes, st, p, v);
    return hipGetLastError();
}

hipError_t launch_penalty_fix(hipStream_t st, const Params &p, const StreamView &v)
{
    hipLaunchKernelGGL((penalty_fix_kernel<kStreamLongR>), dim3((uint32_t)p.B * v.G), dim3(kThreads), 0, st, p, v);
    return hipGetLastError();
}

hipError_t launch_fused(int slice_r, bool pen, uint32_t B, hipStream_t st, const Params &p, const StreamView &v)
{
    const dim3 grid(B * v.G), block(kThreads);
    if (v.list_cap > 2048u) return hipErrorInvalidValue;      // the list lives in static LDS
#define RS_FUSED(Rv) do { if (pen) hipLaunchKernelGGL((fused_kernel<Rv, true>), grid, block, 0, st, p, v);          \
                          else hipLaunchKernelGGL((fused_kernel<Rv, false>), grid, block, 0, st, p, v); } while (0)
    switch (slice_r) {
    case 4:  RS_FUSED(4); break;
    case 8:  RS_FUSED(8); break;
    default: RS_FUSED(16); break;
    }
#undef RS_FUSED
    return hipGetLastError();
}

}  // namespace rs
