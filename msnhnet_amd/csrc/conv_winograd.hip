// Winograd F(2x2,3x3) convolution for 3x3 stride-1 layers (placeholder until the kernels land: every
// entry point reports "unsupported", and algorithm selection never picks it).
#include "common.hpp"

namespace msnh {

size_t winogradWorkspaceBytes(const msnh_conv_desc *) { return 0; }

void winogradPackWeights(const msnh_conv_desc *, const float *, void *) {}

int convWinograd(const msnh_conv_desc *, const void *, const void *, const float *, const float *, const void *, void *, void *,
                 size_t, hipStream_t)
{
    setError("conv2d: the Winograd algorithm is not available in this build");
    return 2;
}

} // namespace msnh
