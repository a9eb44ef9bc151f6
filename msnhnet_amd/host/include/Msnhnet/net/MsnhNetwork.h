// Network (the ordered layer list + its device plan) and NetworkState (per-run state handed to layers).
// Names follow include/Msnhnet/net/MsnhNetwork.h:11-105; the ping-pong memory pools of the reference are
// replaced by the planned device arena owned by `Plan`.
#pragma once
#include <memory>
#include <vector>
#include "Msnhnet/core/MsnhPlan.h"
#include "Msnhnet/layers/MsnhBaseLayer.h"

namespace Msnhnet
{
class NetworkState;

class MsnhNet_API Network
{
public:
    Network() {}
    ~Network() {}
    std::vector<BaseLayer *> layers;
    int batch = 0, height = 0, width = 0, channels = 0, inputNum = 0;
    float *input = nullptr;
    float *output = nullptr;
    std::unique_ptr<Plan> plan;              // valid once weights are loaded
    void forward(NetworkState &netState);    // reference CPU entry point: always throws (no CPU path)
    void forwardGPU(NetworkState &netState); // runs every layer's forwardGPU in order
};

class MsnhNet_API NetworkState
{
public:
    float  *input = nullptr;                 // host pointer of the current batch (NCHW float32)
    int     inputNum = 0;
    Network *net = nullptr;
    int     fixNan = 0;
    msnh_stream_t stream = nullptr;          // stream every layer launches on
    float  *gpuInput = nullptr;              // device copy of `input` (NCHW float32)
};
}
