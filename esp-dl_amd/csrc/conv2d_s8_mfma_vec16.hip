// Instantiations of the int8 implicit-GEMM convolution kernel for operand-B mode B_VEC16.
#include "conv2d_s8_mfma_kernel.h"

namespace espdl {
namespace mfma_conv {

hipError_t launch_vec16(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream)
{
    return pt == 2 ? launch_ksc<B_VEC16, 2>(a, ksc, grid, lds, stream) : launch_ksc<B_VEC16, 1>(a, ksc, grid, lds, stream);
}

} // namespace mfma_conv
} // namespace espdl
