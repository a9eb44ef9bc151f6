// Activation names <-> ActivationType (src/layers/MsnhActivations.cpp:4-60).  The arithmetic itself runs
// in the device epilogues; the host only needs the name table.
#pragma once
#include <string>
#include "Msnhnet/config/MsnhnetCfg.h"

namespace Msnhnet
{
class MsnhNet_API Activations
{
public:
    // Unknown names silently become RELU, exactly like the reference.
    static ActivationType getActivation(const std::string &msg);
    static std::string getActivationStr(const ActivationType &type);
    // true for the activations the device epilogues implement (none, relu, relu6, leaky, mish, swish, logistic)
    static bool deviceSupported(const ActivationType &type);
};
}
