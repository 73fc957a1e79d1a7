// Instantiations of the int8 implicit-GEMM convolution kernel for operand-B mode B_POINT.
#include "conv2d_s8_mfma_kernel.h"

namespace espdl {
namespace mfma_conv {

hipError_t launch_point(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream)
{
    return pt == 2 ? launch_ksc<B_POINT, 2>(a, ksc, grid, lds, stream) : launch_ksc<B_POINT, 1>(a, ksc, grid, lds, stream);
}

} // namespace mfma_conv
} // namespace espdl
