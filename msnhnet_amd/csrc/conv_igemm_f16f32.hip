// Instantiations of the implicit-GEMM convolution kernel for f16 inputs and float outputs (one translation unit per
// type pair so that they compile in parallel).
#include "conv_igemm.hpp"

namespace msnh {
int igemmF16F32(IgemmArgs &a, int groups, int tile, hipStream_t st) { return igemmDispatch<f16, float>(a, groups, tile, st); }
}
