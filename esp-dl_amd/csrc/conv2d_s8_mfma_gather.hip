// Instantiations of the int8 implicit-GEMM convolution kernel for operand-B mode B_GATHER (byte
// gather; only the streamed variant, this mode is the rare fallback).
#include "conv2d_s8_mfma_kernel.h"

namespace espdl {
namespace mfma_conv {

hipError_t launch_gather(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream)
{
    (void)ksc;
    return pt == 2 ? launch_variant<B_GATHER, 2, 0>(a, grid, lds, stream)
                   : launch_variant<B_GATHER, 1, 0>(a, grid, lds, stream);
}

} // namespace mfma_conv
} // namespace espdl
