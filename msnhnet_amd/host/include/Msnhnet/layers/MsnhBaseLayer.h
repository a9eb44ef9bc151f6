// BaseLayer: the layer contract of the host side.  Getter names and the static mode switches follow the
// reference (include/Msnhnet/layers/MsnhBaseLayer.h:17-178); the differences are deliberate:
//   * forward() -- the reference's CPU path -- always throws "Gpu mode , can not run with cpu": this build has
//     no CPU compute path at all;
//   * forwardGPU() launches the layer's slice of the network's device plan (the layer must belong to a network
//     built by NetBuilder, which is where buffers are planned);
//   * lower() is new: it is how a layer describes its computation to the planner.
#pragma once
#include <string>
#include <vector>
#include "Msnhnet/config/MsnhnetCfg.h"
#include "Msnhnet/core/MsnhPlan.h"
#include "Msnhnet/utils/MsnhException.h"
#include "Msnhnet/utils/MsnhTimeUtil.h"

namespace Msnhnet
{
class NetworkState;
class Network;

class MsnhNet_API BaseLayer
{
public:
    BaseLayer();
    virtual ~BaseLayer();

    // process-wide switches, set through NetBuilder before a network is built
    static bool supportAvx;
    static bool supportFma;
    static bool isPreviewMode;
    static bool onlyUseCuda;
    static bool onlyUseCpu;
    static bool onlyUseGpu;
    static bool useFp16;
    static bool convSingleOptim;

    static void setPreviewMode(const bool &isPreviewMode);
    static void setMemAlign(const bool &memAlign);
    static void setForceUseCuda(const bool &forceUseCuda);
    static void setUseFp16(const bool &useFp16);
    static void setOnlyGpu(const bool &onlyGpu);
    static void setOnlyCpu(const bool &onlyCpu);
    static void initSimd();

    virtual void mallocMemory();
    virtual void forward(NetworkState &netState);
    virtual void forwardGPU(NetworkState &netState);
    virtual void loadAllWeigths(std::vector<float> &weights);
    virtual void saveAllWeights(const int &mainIdx, const int &branchIdx = -1, const int &branchIdx1 = -1);

    // Emits this layer's ops into `plan`, reading tensor `in`; returns its output tensor.
    virtual int lower(Plan &plan, int in, int layerIndex);
    // Constants of the ops this layer owns (conv / batchnorm / connected override these).
    virtual const std::vector<float> &kernelWeights() const;
    virtual void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const;
    // The parts this layer's weights consist of, in `.msnhbin` order.  Each part is three numbers: what it is (0 convolution /
    // deconvolution kernel, 1 batch-norm scale, 2 batch-norm shift, 3 running mean, 4 running variance, 5 bias, 6 connected
    // weights), how many floats, and the fan-in of a kernel or connected part.  Lets a caller synthesise a weights file for any graph.
    virtual void weightLayout(std::vector<long long> &parts) const;

    LayerType type() const { return _type; }
    ActivationType activation() const { return _activation; }
    ActivationType getActivation() const { return _activation; }
    int getOutHeight() const { return _outHeight; }
    int getOutWidth() const { return _outWidth; }
    int getOutChannel() const { return _outChannel; }
    int getOutputNum() const { return _outputNum; }
    void setOutHeight(int v) { _outHeight = v; }
    void setOutWidth(int v) { _outWidth = v; }
    void setOutChannel(int v) { _outChannel = v; }
    float *getOutput() const { return nullptr; }            // no host-side activations exist
    float *getGpuOutput() const;                            // device address of this layer's output tensor (NHWC)
    int getInputNum() const { return _inputNum; }
    size_t getWorkSpaceSize() const { return _workSpaceSize; }
    void setWorkSpaceSize(const size_t &v) { _workSpaceSize = v; }
    size_t getNumWeights() const { return _numWeights; }
    std::string getLayerDetail() const { return _layerDetail; }
    int getHeight() const { return _height; }
    int getWidth() const { return _width; }
    int getChannel() const { return _channel; }
    float getForwardTime() const { return _forwardTime; }
    void setForwardTime(float ms) { _forwardTime = ms; }
    std::string getLayerName() const { return _layerName; }
    int getBatch() const { return _batch; }
    size_t getInputSpaceSize() const { return _inputSpaceSize; }
    uint8_t getMemReUse() const { return _memReUse; }
    int getLayerIndex() const { return _layerIndex; }
    void setLayerIndex(int v) { _layerIndex = v; }
    size_t getMaxOutputNum() const { return _maxOutputNum; }
    void setIsBranchLayer(bool v) { _isBranchLayer = v; }
    void setBranchFirst(bool v) { _isFirstBranch = v; }
    void setBranchLast(bool v) { _isLastBranch = v; }
    float getBFlops() const { return _bFlops; }
    bool weightsLoaded() const { return _weightsLoaded; }

    // filled by the planner
    Plan  *plan = nullptr;
    size_t opBegin = 0, opEnd = 0;
    int    outTensor = -1;

protected:
    LayerType      _type = LayerType::EMPTY;
    ActivationType _activation = ActivationType::NONE;
    std::vector<float> _actParams;
    int    _num = 0;
    size_t _workSpaceSize = 0, _inputSpaceSize = 0;
    uint8_t _memReUse = 1;
    bool   _memoryMalloced = false;
    bool   _isBranchLayer = false, _isFirstBranch = false, _isLastBranch = false;
    int    _height = 0, _width = 0, _channel = 0;
    int    _outHeight = 0, _outWidth = 0, _outChannel = 0;
    int    _inputNum = 0, _outputNum = 0;
    size_t _maxOutputNum = 0;
    size_t _numWeights = 0;
    int    _batch = 0;
    float  _bFlops = 0;
    bool   _weightsLoaded = false;
    std::string _layerName = "BaseLayer";
    std::string _layerDetail = "";
    float  _forwardTime = 0;
    int    _layerIndex = 0;

    float actParam() const { return _actParams.empty() ? 0.1f : _actParams[0]; }
    static void requireDeviceActivation(ActivationType act, const char *layer);
};
}
