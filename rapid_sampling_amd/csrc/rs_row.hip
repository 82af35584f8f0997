// Instantiations and the launcher of the row kernel.
#include "rs_row.h"

namespace rs {

template <int R>
static void launch_row_r(int32_t dtype, uint32_t B, hipStream_t st, const Params &p)
{
    if (dtype == RS_DTYPE_F32) hipLaunchKernelGGL((row_kernel<RS_DTYPE_F32, R>), dim3(B), dim3(kRowT), 0, st, p);
    else if (dtype == RS_DTYPE_BF16) hipLaunchKernelGGL((row_kernel<RS_DTYPE_BF16, R>), dim3(B), dim3(kRowT), 0, st, p);
    else hipLaunchKernelGGL((row_kernel<RS_DTYPE_F16, R>), dim3(B), dim3(kRowT), 0, st, p);
}

// groups of four tokens per thread: the fewest of 2, 4, 8, 13 and 16 that hold the row (13: rows of 50304 tokens)
hipError_t launch_row(int32_t dtype, uint32_t B, hipStream_t st, const Params &p)
{
    if (p.V <= 0 || p.V > kRowMaxV || (p.V & 3)) return hipErrorInvalidValue;
    const uint32_t need = (((uint32_t)p.V >> 2) + (uint32_t)kRowW - 1u) / (uint32_t)kRowW;   // groups per wave
    if (need <= 2u * kWave) launch_row_r<2>(dtype, B, st, p);
    else if (need <= 4u * kWave) launch_row_r<4>(dtype, B, st, p);
    else if (need <= 8u * kWave) launch_row_r<8>(dtype, B, st, p);
    else if (need <= 13u * kWave) launch_row_r<13>(dtype, B, st, p);
    else launch_row_r<16>(dtype, B, st, p);
    return hipGetLastError();
}

}  // namespace rs
