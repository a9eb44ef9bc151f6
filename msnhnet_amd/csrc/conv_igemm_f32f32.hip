// Instantiations of the implicit-GEMM convolution kernel for float inputs and float outputs (one translation unit per
// type pair so that they compile in parallel).
#include "conv_igemm.hpp"

namespace msnh {
int igemmF32F32(IgemmArgs &a, int groups, int tile, hipStream_t st) { return igemmDispatch<float, float>(a, groups, tile, st); }
}
