// Instantiations and launchers of the cluster kernels.
#include "rs_cluster.h"

namespace rs {

template <bool PEN>
static hipError_t launch_sample_t(int R, dim3 grid, hipStream_t st, const Params &p)
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

hipError_t launch_sample(bool pen, int R, dim3 grid, hipStream_t st, const Params &p)
{
    return pen ? launch_sample_t<true>(R, grid, st, p) : launch_sample_t<false>(R, grid, st, p);
}

}  // namespace rs
