// Compile-time configuration and the enumerations shared by parser, layers and the C facade.
// Numeric values of ActivationType / LayerType equal the reference's
// (include/Msnhnet/config/MsnhnetCfg.h:95-157) so integer values stored by callers keep their meaning.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#ifndef MsnhNet_API
#define MsnhNet_API __attribute__((visibility("default")))
#endif

namespace Msnhnet
{
enum ActivationType
{
    LOGISTIC = 0, RELU, RELU6, RELIE, RAMP, TANH, PRELU, PLSE, LEAKY, ELU, LOGGY, STAIR, HARDTAN, LHTAN,
    SOFT_PLUS, SELU, SWISH, HARD_SWISH, MISH, NORM_CHAN, NORM_CHAN_SOFTMAX, NORM_CHAN_SOFTMAX_MAXVAL, NONE
};

enum LayerType
{
    CONVOLUTIONAL = 0, DECONVOLUTIONAL, CONNECTED, MAXPOOL, LOCAL_AVGPOOL, GLOBAL_AVGPOOL, SOFTMAX, CROP, ROUTE,
    VARIABLE_OP, NORMALIZATION, AVGPOOL, ACTIVE, BATCHNORM, NETWORK, YOLO, YOLO_OUT, GAUSSIAN_YOLO, UPSAMPLE,
    L2NORM, EMPTY, VIEW, PERMUTE, PIXEL_SHUFFLE, SLICE, REDUCTION, CONFIG, RES_BLOCK, RES_2_BLOCK, CONCAT_BLOCK,
    ADD_BLOCK, PADDING, CLIP
};
}
