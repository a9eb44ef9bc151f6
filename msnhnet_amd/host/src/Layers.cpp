// Layer classes: shape inference, weight slicing and lowering into plan ops.
// Shape rules, weight order and exception texts follow the reference's layer sources (cited per class in
// MsnhLayers.h); none of its compute code exists here -- the arithmetic lives in the device kernels.
#include "Msnhnet/layers/MsnhLayers.h"
#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include "Msnhnet/net/MsnhNetwork.h"
#include "Msnhnet/utils/MsnhExVector.h"
#include "Msnhnet/utils/MsnhTaskPool.h"

namespace Msnhnet
{
// ---- BaseLayer -------------------------------------------------------------------------------------------------
bool BaseLayer::supportAvx = false;
bool BaseLayer::supportFma = false;
bool BaseLayer::isPreviewMode = false;
bool BaseLayer::onlyUseCuda = false;
bool BaseLayer::onlyUseCpu = false;
bool BaseLayer::onlyUseGpu = true;          // there is no CPU compute path in this build
bool BaseLayer::useFp16 = false;
bool BaseLayer::convSingleOptim = false;

BaseLayer::BaseLayer() {}
BaseLayer::~BaseLayer() {}
void BaseLayer::setPreviewMode(const bool &v) { isPreviewMode = v; }
void BaseLayer::setMemAlign(const bool &) {}
void BaseLayer::setForceUseCuda(const bool &v) { onlyUseCuda = v; }
void BaseLayer::setUseFp16(const bool &v) { useFp16 = v; }
void BaseLayer::setOnlyGpu(const bool &v) { onlyUseGpu = v; }
void BaseLayer::setOnlyCpu(const bool &v) { onlyUseCpu = v; }
void BaseLayer::initSimd() {}
void BaseLayer::mallocMemory() { _memReUse = 0; _memoryMalloced = true; }

void BaseLayer::forward(NetworkState &)
{
    MSNH_THROW("Gpu mode , can not run with cpu");
}

void BaseLayer::forwardGPU(NetworkState &netState)
{
    if (plan == nullptr) MSNH_THROW(_layerName + ": layer is not part of a planned network (build it with NetBuilder and load weights first)");
    plan->run(opBegin, opEnd, netState.stream);
}

void BaseLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (!weights.empty()) MSNH_THROW(_layerName + " has no weights");
}

void BaseLayer::saveAllWeights(const int &, const int &, const int &) {}

void BaseLayer::weightLayout(std::vector<long long> &) const {}

static void addPart(std::vector<long long> &parts, int what, long long count, long long fanIn = 0)
{
    if (count <= 0) return;
    parts.push_back(what); parts.push_back(count); parts.push_back(fanIn);
}

int BaseLayer::lower(Plan &, int, int) { MSNH_THROW(_layerName + ": lowering is not implemented"); }

const std::vector<float> &BaseLayer::kernelWeights() const
{
    static const std::vector<float> none;
    return none;
}

void BaseLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.clear();
    shift.clear();
}

float *BaseLayer::getGpuOutput() const
{
    if (plan == nullptr || outTensor < 0) return nullptr;
    return static_cast<float *>(plan->ptr(outTensor));
}

void BaseLayer::requireDeviceActivation(ActivationType act, const char *layer)
{
    if (!Activations::deviceSupported(act))
        MSNH_THROW(std::string(layer) + ": activation '" + Activations::getActivationStr(act) + "' is outside the convolutional path this build implements");
}

static std::string fmt(const char *f, ...)
{
    char buf[256];
    va_list ap;
    va_start(ap, f);
    vsnprintf(buf, sizeof(buf), f, ap);
    va_end(ap);
    return buf;
}

static int planDtype(const Plan &plan) { return plan.computeDtype; }

// Batch-norm folded the way the reference evaluates it (src/layers/MsnhConvolutionalLayer.cpp:811-815):
// sqrtVal = sqrt(var+eps); scale = gamma/sqrtVal; shift = -gamma*mean/sqrtVal + beta, all in float.
static void foldBn(const std::vector<float> &g, const std::vector<float> &beta, const std::vector<float> &mean, const std::vector<float> &var,
                   float eps, std::vector<float> &scale, std::vector<float> &shift)
{
    const size_t n = g.size();
    scale.resize(n);
    shift.resize(n);
    for (size_t c = 0; c < n; ++c)
    {
        const float sqrtVal = static_cast<float>(std::sqrt(var[c] + eps));
        const float scaleSqrt = g[c] / sqrtVal;
        const float meanSqrt = -g[c] * mean[c] / sqrtVal;
        scale[c] = scaleSqrt;
        shift[c] = meanSqrt + (beta.empty() ? 0.f : beta[c]);
    }
}

// ---- ConvolutionalLayer -------------------------------------------------------------------------------------------
ConvolutionalLayer::ConvolutionalLayer(const int &batch, const int &steps, const int &height, const int &width, const int &channel, const int &num,
                                       const int &groups, const int &kSizeX, const int &kSizeY, const int &strideX, const int &strideY,
                                       const int &dilationX, const int &dilationY, const int &paddingX, const int &paddingY,
                                       ActivationType activation, const std::vector<float> &actParams, const int &batchNorm, const float &bnEps,
                                       const int &useBias, const int &binary, const int &xnor, const int &useBinOutput, const int &groupIndex,
                                       const int &antialiasing, ConvolutionalLayer *const &shareLayer, const int &assistedExcitation, const int &deform)
{
    (void)steps; (void)useBinOutput; (void)groupIndex; (void)deform;
    if (binary || xnor || shareLayer != nullptr || assistedExcitation || antialiasing)
        MSNH_THROW("conv: binary/xnor/shared/assisted-excitation/antialiasing variants are outside the convolutional path this build implements");
    if (activation == ActivationType::PRELU || activation == NORM_CHAN || activation == NORM_CHAN_SOFTMAX || activation == NORM_CHAN_SOFTMAX_MAXVAL)
        MSNH_THROW("conv: prelu / channel-normalising activations are outside the convolutional path this build implements");
    requireDeviceActivation(activation, "conv");
    _type = LayerType::CONVOLUTIONAL;
    _groups = groups < 1 ? 1 : groups;
    _strideX = strideX; _strideY = strideY;
    _height = height; _width = width; _channel = channel; _num = num; _batch = batch;
    _dilationX = dilationX; _dilationY = dilationY; _kSizeX = kSizeX; _kSizeY = kSizeY; _paddingX = paddingX; _paddingY = paddingY;
    _batchNorm = batchNorm; _useBias = useBias; _bnEps = bnEps;
    if (num <= 0 || kSizeX <= 0 || kSizeY <= 0 || strideX <= 0 || strideY <= 0) MSNH_THROW("conv: filters, kSize and stride must be positive");
    if (channel % _groups != 0 || num % _groups != 0) MSNH_THROW("conv: channels and filters must be divisible by groups");
    // The reference feeds X-named sizes into the H slots of its im2col while the output size uses Y for the height
    // (src/layers/MsnhConvolutionalLayer.cpp:750-752 vs :388-398), so only square geometry is self-consistent there.
    if (kSizeX != kSizeY || strideX != strideY || paddingX != paddingY || dilationX != dilationY)
        MSNH_THROW("conv: only square kernels / strides / paddings / dilations are supported");
    _nWeights = (channel / groups) * num * kSizeX * kSizeY;
    _nBiases = useBias ? num : 0;
    if (batchNorm) { _nScales = num; _nRollMean = num; _nRollVariance = num; }
    _outHeight = convOutHeight();
    _outWidth = convOutWidth();
    _outChannel = num;
    if (_outHeight <= 0 || _outWidth <= 0) MSNH_THROW("conv: kernel larger than the padded input");
    _outputNum = _outHeight * _outWidth * _outChannel;
    _inputNum = height * width * channel;
    _activation = activation;
    _actParams = actParams;
    _numWeights = static_cast<size_t>(_nWeights + _nScales + _nRollMean + _nRollVariance + _nBiases);
    _workSpaceSize = 0;                       // implicit GEMM: no im2col scratch
    _inputSpaceSize = static_cast<size_t>(_inputNum);
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _bFlops = (2.0f * _nWeights * _outHeight * _outWidth) / 1000000000.f;

    const char *tag = "conv  ";
    _layerName = "Conv            ";
    if (_batchNorm) { _layerName = "ConvBN          "; tag = "convBN"; }
    else if (_groups == _num) { _layerName = "ConvDW          "; tag = "convDW"; }
    _layerDetail = tag;
    _layerDetail += _groups > 1 ? fmt("%5d/%4d ", _num, _groups) : fmt("%5d      ", _num);
    _layerDetail += _dilationX > 1 ? fmt("%2d x%2d/%2d(%1d)", _kSizeX, _kSizeY, _strideX, _dilationX) : fmt("%2d x%2d/%2d   ", _kSizeX, _kSizeY, _strideX);
    _layerDetail += fmt("%4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _width, _height, _channel, _outWidth, _outHeight, _outChannel,
                        static_cast<double>(_bFlops));
}

int ConvolutionalLayer::convOutHeight() const { return (_height + 2 * _paddingY - (_dilationY * (_kSizeY - 1) + 1)) / _strideY + 1; }
int ConvolutionalLayer::convOutWidth() const { return (_width + 2 * _paddingX - (_dilationX * (_kSizeX - 1) + 1)) / _strideX + 1; }

void ConvolutionalLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (weights.size() != _numWeights)
        MSNH_THROW("Conv weights load err. needed : " + std::to_string(_numWeights) + " given : " + std::to_string(weights.size()));
    if (BaseLayer::isPreviewMode) return;
    const float *p = weights.data();
    _weights.assign(p, p + _nWeights);
    p += _nWeights;
    if (_batchNorm)
    {
        // order: scales, biases (only when useBias), rollMean, rollVariance  (src/layers/MsnhConvolutionalLayer.cpp:1275-1288)
        _scales.assign(p, p + _nScales); p += _nScales;
        _biases.assign(p, p + _nBiases); p += _nBiases;
        _rollMean.assign(p, p + _nRollMean); p += _nRollMean;
        _rollVariance.assign(p, p + _nRollVariance);
    }
    else if (_useBias)
    {
        _biases.assign(p, p + _nBiases);
    }
    _weightsLoaded = true;
}

void ConvolutionalLayer::weightLayout(std::vector<long long> &parts) const
{
    addPart(parts, 0, _nWeights, static_cast<long long>(_channel / _groups) * _kSizeX * _kSizeY);
    if (_batchNorm)
    {
        addPart(parts, 1, _nScales); addPart(parts, 2, _nBiases); addPart(parts, 3, _nRollMean); addPart(parts, 4, _nRollVariance);
    }
    else if (_useBias) addPart(parts, 5, _nBiases, static_cast<long long>(_channel / _groups) * _kSizeX * _kSizeY);
}

void ConvolutionalLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.clear();
    shift.clear();
    if (_batchNorm) foldBn(_scales, _biases, _rollMean, _rollVariance, _bnEps, scale, shift);
    else if (_useBias) shift = _biases;
}

int ConvolutionalLayer::lower(Plan &plan, int in, int layerIndex)
{
    const int dtype = planDtype(plan);
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, dtype, "conv_out");
    if (plan.tensors[static_cast<size_t>(in)].layout == PlanTensor::NCHW_INPUT)
    {
        // first layer: use the stem kernel (reads the NCHW float32 input directly) when the shape allows it
        msnh_conv_desc d;
        std::memset(&d, 0, sizeof(d));
        d.dtype = dtype; d.out_dtype = dtype; d.batch = _batch; d.in_h = _height; d.in_w = _width; d.in_c = _channel; d.in_ld = _channel;
        d.out_c = _outChannel; d.out_h = _outHeight; d.out_w = _outWidth; d.out_ld = (_outChannel + 7) / 8 * 8;
        d.ksize = _kSizeX; d.stride = _strideX; d.pad = _paddingX; d.dilation = _dilationX; d.groups = _groups;
        d.act = NONE; d.act2 = NONE; d.res_ld = d.out_c; d.res_mul = 1.f; d.out_mul = 1.f; d.algo = MSNH_CONV_AUTO;
        if (msnh_hip_conv2d_select_algo(&d) != MSNH_CONV_STEM)
        {
            const int cast = plan.addTensor(_batch, _height, _width, _channel, dtype, "input_nhwc");
            plan.addOp(PlanOp::INPUT_CAST, in, -1, cast, layerIndex, "input_cast");
            in = cast;
        }
    }
    PlanOp &op = plan.addOp(PlanOp::CONV, in, -1, out, layerIndex, "conv");
    op.ksize = _kSizeX; op.stride = _strideX; op.pad = _paddingX; op.dilation = _dilationX; op.groups = _groups;
    op.act = _activation; op.actParam = actParam();
    op.src = this;
    return out;
}

// ---- BatchNormLayer --------------------------------------------------------------------------------------------------
BatchNormLayer::BatchNormLayer(const int &batch, const int &width, const int &height, const int &channel, const ActivationType &activation,
                               const float &eps, const std::vector<float> &actParams)
{
    requireDeviceActivation(activation, "batchnorm");
    _type = LayerType::BATCHNORM;
    _layerName = "BatchNorm       ";
    _activation = activation;
    _actParams = actParams;
    _eps = eps;
    _batch = batch; _width = width; _height = height; _channel = channel;
    _outWidth = width; _outHeight = height; _outChannel = channel;
    _num = channel;
    _inputNum = width * height * channel;
    _outputNum = _inputNum;
    _numWeights = static_cast<size_t>(4) * channel;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("Batch Normalization Layer:     %d x %d x %d image\n", _width, _height, _channel);
}

void BatchNormLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (weights.size() != _numWeights)
        MSNH_THROW("BatchNorm weights load err. needed : " + std::to_string(_numWeights) + " given : " + std::to_string(weights.size()));
    if (BaseLayer::isPreviewMode) return;
    const float *p = weights.data();
    const int c = _channel;
    _scales.assign(p, p + c);               // scales, biases, rollMean, rollVariance (src/layers/MsnhBatchNormLayer.cpp:469-472)
    _biases.assign(p + c, p + 2 * c);
    _rollMean.assign(p + 2 * c, p + 3 * c);
    _rollVariance.assign(p + 3 * c, p + 4 * c);
    _weightsLoaded = true;
}

void BatchNormLayer::weightLayout(std::vector<long long> &parts) const
{
    for (int what = 1; what <= 4; ++what) addPart(parts, what, _channel);
}

void BatchNormLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    foldBn(_scales, _biases, _rollMean, _rollVariance, _eps, scale, shift);
}

int BatchNormLayer::lower(Plan &plan, int in, int layerIndex)
{
    const PlanTensor &ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout != PlanTensor::NHWC) MSNH_THROW("batchnorm can not be the first layer of a network");
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, planDtype(plan), "bn_out");
    PlanOp &op = plan.addOp(PlanOp::AFFINE, in, -1, out, layerIndex, "batchnorm");
    op.act = _activation; op.actParam = actParam();
    op.src = this;
    return out;
}

// ---- pooling ------------------------------------------------------------------------------------------------------------
static int pooledSize(int in, int k, int s, int p, int ceilMode, const char *name)
{
    if (ceilMode == 1)
    {
        const int rem = (in + p * 2 - k) % s;
        if (rem >= k) MSNH_THROW(std::string(name) + " padding error ");
        return (in + p * 2 - k) / s + (rem <= p ? 1 : 2);
    }
    if (ceilMode == 0) return (in + p * 2 - k) / s + 1;
    return (in + p - k) / s + 1;
}

MaxPoolLayer::MaxPoolLayer(const int &batch, const int &height, const int &width, const int &channel, const int &kSizeX, const int &kSizeY,
                           const int &strideX, const int &strideY, const int &paddingX, const int &paddingY, const int &maxPoolDepth,
                           const int &outChannelsMp, const int &ceilMode, const int &antialiasing)
    : _kSizeX(kSizeX), _kSizeY(kSizeY), _strideX(strideX), _strideY(strideY), _paddingX(paddingX), _paddingY(paddingY), _ceilMode(ceilMode)
{
    (void)outChannelsMp; (void)antialiasing;
    if (maxPoolDepth) MSNH_THROW("maxpool: depth mode is outside the convolutional path this build implements");
    if (kSizeX != kSizeY || strideX != strideY || paddingX != paddingY) MSNH_THROW("maxpool: only square windows are supported");
    if (kSizeX <= 0 || strideX <= 0) MSNH_THROW("maxpool: kSize and stride must be positive");
    _type = LayerType::MAXPOOL;
    _layerName = "MaxPool         ";
    _batch = batch; _height = height; _width = width; _channel = channel;
    _outWidth = pooledSize(width, kSizeX, strideX, paddingX, ceilMode, "maxpool");
    _outHeight = pooledSize(height, kSizeY, strideY, paddingY, ceilMode, "maxpool");
    _outChannel = channel;
    _outputNum = _outHeight * _outWidth * _outChannel;
    _inputNum = height * width * channel;
    _bFlops = (_kSizeX * _kSizeY * _channel * _outHeight * _outWidth) / 1000000000.f;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("max               %2dx%2d/%2d   %4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _kSizeX, _kSizeY, _strideX, _width, _height,
                       _channel, _outWidth, _outHeight, _outChannel, static_cast<double>(_bFlops));
}

int MaxPoolLayer::lower(Plan &plan, int in, int layerIndex)
{
    if (plan.tensors[static_cast<size_t>(in)].layout != PlanTensor::NHWC) MSNH_THROW("maxpool can not be the first layer of a network");
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, plan.tensors[static_cast<size_t>(in)].dtype, "maxpool_out");
    PlanOp &op = plan.addOp(PlanOp::MAXPOOL, in, -1, out, layerIndex, "maxpool");
    op.ksize = _kSizeX; op.stride = _strideX; op.pad = _paddingX;
    return out;
}

LocalAvgPoolLayer::LocalAvgPoolLayer(const int &batch, const int &height, const int &width, const int &channel, const int &kSizeX, const int &kSizeY,
                                     const int &strideX, const int &strideY, const int &paddingX, const int &paddingY, const int &ceilMode,
                                     const int &antialiasing)
    : _kSizeX(kSizeX), _kSizeY(kSizeY), _strideX(strideX), _strideY(strideY), _paddingX(paddingX), _paddingY(paddingY), _ceilMode(ceilMode)
{
    (void)antialiasing;
    if (kSizeX != kSizeY || strideX != strideY || paddingX != paddingY) MSNH_THROW("localavgpool: only square windows are supported");
    if (kSizeX <= 0 || strideX <= 0) MSNH_THROW("localavgpool: kSize and stride must be positive");
    _type = LayerType::LOCAL_AVGPOOL;
    _layerName = "LocalAvgPool    ";
    _batch = batch; _height = height; _width = width; _channel = channel;
    _outWidth = pooledSize(width, kSizeX, strideX, paddingX, ceilMode, "localavgpool");
    _outHeight = pooledSize(height, kSizeY, strideY, paddingY, ceilMode, "localavgpool");
    _outChannel = channel;
    _outputNum = _outHeight * _outWidth * _outChannel;
    _inputNum = height * width * channel;
    _bFlops = (_kSizeX * _kSizeY * _channel * _outHeight * _outWidth) / 1000000000.f;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("avg               %2dx%2d/%2d   %4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _kSizeX, _kSizeY, _strideX, _width, _height,
                       _channel, _outWidth, _outHeight, _outChannel, static_cast<double>(_bFlops));
}

int LocalAvgPoolLayer::lower(Plan &plan, int in, int layerIndex)
{
    if (plan.tensors[static_cast<size_t>(in)].layout != PlanTensor::NHWC) MSNH_THROW("localavgpool can not be the first layer of a network");
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, plan.tensors[static_cast<size_t>(in)].dtype, "avgpool_out");
    PlanOp &op = plan.addOp(PlanOp::AVGPOOL, in, -1, out, layerIndex, "localavgpool");
    op.ksize = _kSizeX; op.stride = _strideX; op.pad = _paddingX;
    return out;
}

// ---- ConnectedLayer ---------------------------------------------------------------------------------------------------------
ConnectedLayer::ConnectedLayer(const int &batch, const int &steps, const int &inputNum, const int &outputNum, const ActivationType &activation,
                               const std::vector<float> &actParams, const int &batchNorm, const float &bnEps, const int &useBias)
{
    (void)steps; (void)bnEps;
    if (batchNorm) MSNH_THROW("connect: batchNorm is outside the convolutional path this build implements");
    requireDeviceActivation(activation, "connect");
    if (inputNum <= 0 || outputNum <= 0) MSNH_THROW("connect: input and output sizes must be positive");
    _type = LayerType::CONNECTED;
    _layerName = "Connected       ";
    _inputNum = inputNum; _outputNum = outputNum; _batch = batch; _batchNorm = batchNorm;
    _height = 1; _width = 1; _channel = inputNum;
    _outHeight = 1; _outWidth = 1; _outChannel = outputNum; _num = outputNum;
    _activation = activation; _actParams = actParams; _useBias = useBias;
    _nWeights = inputNum * outputNum;
    _nBiases = useBias ? outputNum : 0;
    _numWeights = static_cast<size_t>(_nWeights + _nBiases);
    _inputSpaceSize = static_cast<size_t>(_inputNum);
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("connected                            %4d  ->  %4d\n", inputNum, outputNum);
}

void ConnectedLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (weights.size() != _numWeights)
        MSNH_THROW("Connect weights load err. needed : " + std::to_string(_numWeights) + " given : " + std::to_string(weights.size()));
    if (BaseLayer::isPreviewMode) return;
    _weights.assign(weights.begin(), weights.begin() + _nWeights);
    if (_useBias) _biases.assign(weights.begin() + _nWeights, weights.end());
    _weightsLoaded = true;
}

void ConnectedLayer::weightLayout(std::vector<long long> &parts) const
{
    addPart(parts, 6, _nWeights, _inputNum);
    if (_useBias) addPart(parts, 5, static_cast<long long>(_numWeights) - _nWeights, _inputNum);
}

void ConnectedLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.clear();
    shift = _biases;
}

int ConnectedLayer::lower(Plan &plan, int in, int layerIndex)
{
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout == PlanTensor::NCHW_INPUT) MSNH_THROW("connect can not be the first layer of a network");
    // (an image tensor with more than one pixel is flattened in the reference's channel-major order: the weights are permuted to
    //  the device's pixel-major order when they are uploaded, Plan::prepareWeights)
    // keep the classifier tail in float32: an average pool feeding the classifier writes float32
    const int p = plan.producerOf(in);
    if (p >= 0 && plan.ops[static_cast<size_t>(p)].kind == PlanOp::AVGPOOL && plan.consumerCount(in) == 0)
        plan.tensors[static_cast<size_t>(in)].dtype = MSNH_F32;
    const int out = plan.addTensor(_batch, 1, 1, _outputNum, MSNH_F32, "connected_out", PlanTensor::FLAT);
    PlanOp &op = plan.addOp(PlanOp::CONNECTED, in, -1, out, layerIndex, "connected");
    op.act = _activation; op.actParam = actParam();
    op.src = this;
    return out;
}

// ---- UpSample / Empty / Route ---------------------------------------------------------------------------------------------------
UpSampleLayer::UpSampleLayer(const int &batch, const int &width, const int &height, const int &channel, const int &strideX, const int &strideY,
                             const float &scaleX, const float &scaleY, UpSampleParams::UpsampleType upsampleType, const int &alignCorners)
    : _strideX(strideX), _strideY(strideY), _scaleX(scaleX), _scaleY(scaleY), _upsampleType(upsampleType), _alignCorners(alignCorners)
{
    _type = LayerType::UPSAMPLE;
    _layerName = "UpSample        ";
    _batch = batch; _width = width; _height = height; _channel = channel;
    if (upsampleType == UpSampleParams::NEAREST)
    {
        if (strideX != strideY || strideX <= 0) MSNH_THROW("upsample: strideX and strideY must be equal and positive");
        _outWidth = width * strideX; _outHeight = height * strideY;
    }
    else
    {
        // src/layers/MsnhUpSampleLayer.cpp:20-24
        _outWidth = static_cast<int>(width * scaleX); _outHeight = static_cast<int>(height * scaleY);
        if (_outWidth < 1 || _outHeight < 1) MSNH_THROW("w*x and outw*outx must > 1");
    }
    _outChannel = channel;
    _outputNum = _outWidth * _outHeight * _outChannel;
    _inputNum = width * height * channel;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    if (upsampleType == UpSampleParams::NEAREST)
        _layerDetail = fmt("upsample              %2dx%2d  %4d x%4d x%4d -> %4d x%4d x%4d\n", _strideX, _strideY, _width, _height, _channel, _outHeight,
                           _outHeight, _outChannel);
    else
        _layerDetail = fmt("upsample          %4fx%4f  %4d x%4d x%4d -> %4d x%4d x%4d\n", _scaleX, _scaleY, _width, _height, _channel, _outHeight,
                           _outHeight, _outChannel);
}

int UpSampleLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, plan.tensors[static_cast<size_t>(in)].dtype, "upsample_out");
    if (_upsampleType == UpSampleParams::BILINEAR)
    {
        PlanOp &op = plan.addOp(PlanOp::BILINEAR, in, -1, out, layerIndex, "upsample_bilinear");
        op.alignCorners = _alignCorners;
        return out;
    }
    PlanOp &op = plan.addOp(PlanOp::UPSAMPLE, in, -1, out, layerIndex, "upsample");
    op.stride = _strideX;
    op.upScale = _scaleX;          // Blas::cpuUpSample is called with scaleX only (src/layers/MsnhUpSampleLayer.cpp:106)
    return out;
}

// ---- DeConvolutionalLayer -----------------------------------------------------------------------------------------------
namespace
{
// weights of the 1x1 convolution a transposed convolution lowers to; no affine of its own
class DeconvGemmWeights : public BaseLayer
{
public:
    std::vector<float> w;
    const std::vector<float> &kernelWeights() const override { return w; }
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override { scale.clear(); shift.clear(); }
};
}

DeConvolutionalLayer::DeConvolutionalLayer(const int &batch, const int &height, const int &width, const int &channel, const int &num, const int &kSizeX,
                                           const int &kSizeY, const int &strideX, const int &strideY, const int &paddingX, const int &paddingY,
                                           const int &groups, const ActivationType &activation, const std::vector<float> &actParams, const int &useBias)
    : _kSizeX(kSizeX), _kSizeY(kSizeY), _strideX(strideX), _strideY(strideY), _paddingX(paddingX), _paddingY(paddingY), _useBias(useBias)
{
    requireDeviceActivation(activation, "deconv");
    if (groups > 1) MSNH_THROW("deconv: groups are outside the convolutional path this build implements");
    if (kSizeX != kSizeY || strideX != strideY || paddingX != paddingY) MSNH_THROW("deconv: only square kernels, strides and paddings are supported");
    if (kSizeX <= 0 || strideX <= 0 || paddingX < 0 || num <= 0) MSNH_THROW("deconv: bad geometry");
    _type = LayerType::DECONVOLUTIONAL;
    _layerName = "DeConv          ";
    _batch = batch; _height = height; _width = width; _channel = channel; _num = num;
    _activation = activation; _actParams = actParams;
    _outHeight = deConvOutHeight(); _outWidth = deConvOutWidth(); _outChannel = num;
    if (_outHeight <= 0 || _outWidth <= 0) MSNH_THROW("deconv: non-positive output size");
    _outputNum = _outWidth * _outHeight * _outChannel;
    _inputNum = width * width * channel;                                 // (sic, src/layers/MsnhDeConvolutionalLayer.cpp:46)
    _nWeights = channel * num * kSizeX * kSizeY;
    _nBiases = useBias ? num : 0;
    _numWeights = static_cast<size_t>(_nWeights + _nBiases);
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("Deconvolutional Layer: %d x %d x %d image, %d filters -> %d x %d x %d image\n", _height, _width, _channel, _num, _outHeight,
                       _outWidth, _num);
    _gemm = new DeconvGemmWeights();
}

DeConvolutionalLayer::~DeConvolutionalLayer() { delete _gemm; }

void DeConvolutionalLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (weights.size() != _numWeights)
        MSNH_THROW("Deconv weights load err. needed : " + std::to_string(_numWeights) + " given : " + std::to_string(weights.size()));
    if (BaseLayer::isPreviewMode) return;
    // file order [channel][filters][ky][kx] -> rows of the 1x1 convolution [(ky*k + kx)*filters + oc][channel]
    const int kk = _kSizeX * _kSizeY;
    std::vector<float> &w = static_cast<DeconvGemmWeights *>(_gemm)->w;
    w.assign(static_cast<size_t>(_nWeights), 0.f);
    for (int ic = 0; ic < _channel; ++ic)
        for (int oc = 0; oc < _num; ++oc)
            for (int t = 0; t < kk; ++t)
                w[(static_cast<size_t>(t) * _num + oc) * _channel + ic] = weights[(static_cast<size_t>(ic) * _num + oc) * kk + t];
    if (_useBias) _biases.assign(weights.begin() + _nWeights, weights.end());
    _weightsLoaded = true;
}

void DeConvolutionalLayer::weightLayout(std::vector<long long> &parts) const
{
    addPart(parts, 0, _nWeights, static_cast<long long>(_channel) * _kSizeX * _kSizeY);
    if (_useBias) addPart(parts, 5, static_cast<long long>(_numWeights) - _nWeights, static_cast<long long>(_channel) * _kSizeX * _kSizeY);
}

void DeConvolutionalLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.clear();
    shift = _biases;
}

int DeConvolutionalLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout != PlanTensor::NHWC) MSNH_THROW("Layer before deconvolutional layer must output image");
    const int kk = _kSizeX * _kSizeY;
    const int cols = plan.addTensor(ti.n, ti.h, ti.w, kk * _num, ti.dtype, "deconv_cols");
    PlanOp &gemm = plan.addOp(PlanOp::CONV, in, -1, cols, layerIndex, "deconv_gemm");
    gemm.ksize = 1; gemm.stride = 1; gemm.pad = 0; gemm.dilation = 1; gemm.groups = 1;
    gemm.src = _gemm;
    const int out = plan.addTensor(ti.n, _outHeight, _outWidth, _num, ti.dtype, "deconv_out");
    PlanOp &op = plan.addOp(PlanOp::COL2IM, cols, -1, out, layerIndex, "deconv_col2im");
    op.ksize = _kSizeX; op.stride = _strideX; op.pad = _paddingX;
    op.act = _activation; op.actParam = actParam();
    op.src = this;
    return out;
}

GlobalAvgPoolLayer::GlobalAvgPoolLayer(const int &batch, const int &height, const int &width, const int &channel)
{
    _type = LayerType::GLOBAL_AVGPOOL;
    _layerName = "GlobalAvgPool   ";
    _batch = batch; _height = height; _width = width; _channel = channel;
    _outWidth = 1; _outHeight = 1; _outChannel = channel;
    _inputNum = height * width * channel;
    _outputNum = channel;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("GlobalAvgPool                %4d x%4d x%4d ->   %4d\n", _width, _height, _channel, _outChannel);
}

int GlobalAvgPoolLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout != PlanTensor::NHWC) MSNH_THROW("globalavgpool: the input must be an image tensor");
    const int out = plan.addTensor(ti.n, 1, 1, ti.c, ti.dtype, "globalavgpool_out");
    // the local average pool divides by the number of valid window elements: a window covering the whole plane is the global mean
    PlanOp &op = plan.addOp(PlanOp::AVGPOOL, in, -1, out, layerIndex, "globalavgpool");
    op.ksize = std::max(ti.h, ti.w); op.stride = 1; op.pad = 0;
    return out;
}

SoftMaxLayer::SoftMaxLayer(const int &batch, const int &inputNum, const int &groups, const float &temperature)
    : _groups(groups), _temperature(temperature)
{
    if (groups != 1) MSNH_THROW("softmax: groups are outside the convolutional path this build implements");
    if (temperature == 0.f) MSNH_THROW("softmax: temperature must not be 0");
    _type = LayerType::SOFTMAX;
    _layerName = "SoftMax         ";
    _batch = batch;
    _inputNum = inputNum; _outputNum = inputNum;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("softmax                                        %4d\n", inputNum);
}

int SoftMaxLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    _outHeight = ti.h; _outWidth = ti.w; _outChannel = ti.c;
    const int out = plan.addTensor(ti.n, ti.h, ti.w, ti.c, ti.dtype, "softmax_out", ti.layout);
    PlanOp &op = plan.addOp(PlanOp::SOFTMAX, in, -1, out, layerIndex, "softmax");
    op.upScale = _temperature;
    return out;
}

// ---- stand-alone activation / padding / slice / variable op --------------------------------------------------------------------
ActivationLayer::ActivationLayer(const int &batch, const int &width, const int &height, const int &channel, const int &inputNum,
                                 const ActivationType &activation, const std::vector<float> &actParams)
{
    if (activation == ActivationType::PRELU) MSNH_THROW("act: prelu is outside the convolutional path this build implements");
    requireDeviceActivation(activation, "act");
    _type = LayerType::ACTIVE;
    _layerName = "Activate        ";
    _batch = batch; _width = width; _height = height; _channel = channel;
    _outWidth = width; _outHeight = height; _outChannel = channel;
    _inputNum = inputNum; _outputNum = inputNum;
    _activation = activation; _actParams = actParams;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = "Activate Layer: " + Activations::getActivationStr(activation) + "\n";
}

void ActivationLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.assign(static_cast<size_t>(_channel), 1.f);
    shift.assign(static_cast<size_t>(_channel), 0.f);
}

int ActivationLayer::lower(Plan &plan, int in, int layerIndex)
{
    if (_activation == ActivationType::NONE) return in;          // identity: the reference copies, the plan aliases
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    // (the flat float32 vector a connected layer writes is a 1 x 1 image of `outputs` channels to the element-wise kernel)
    const int out = plan.addTensor(ti.n, ti.h, ti.w, ti.c, ti.dtype, "act_out", ti.layout);
    PlanOp &op = plan.addOp(PlanOp::AFFINE, in, -1, out, layerIndex, "act");
    op.act = _activation; op.actParam = actParam();
    op.pureAct = true;
    op.src = this;
    return out;
}

PaddingLayer::PaddingLayer(const int &batch, const int &height, const int &width, const int &channel, const int &top, const int &down,
                           const int &left, const int &right, const float &paddingVal)
    : _top(top), _down(down), _left(left), _right(right), _paddingVal(paddingVal)
{
    if (top < 0 || down < 0 || left < 0 || right < 0) MSNH_THROW("padding: negative padding");
    _type = LayerType::PADDING;
    _layerName = "Padding         ";
    _batch = batch; _height = height; _width = width; _channel = channel;
    _inputNum = width * height * channel;
    _outHeight = height + top + down; _outWidth = width + left + right; _outChannel = channel;
    _outputNum = _outHeight * _outWidth * _outChannel;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("Padding                      %4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _width, _height, _channel, _outWidth, _outHeight,
                       _outChannel, 0.0);
}

int PaddingLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout != PlanTensor::NHWC) MSNH_THROW("padding: the input must be an image tensor");
    const int out = plan.addTensor(ti.n, _outHeight, _outWidth, ti.c, ti.dtype, "padding_out");
    PlanOp &op = plan.addOp(PlanOp::PAD, in, -1, out, layerIndex, "padding");
    op.padTop = _top; op.padLeft = _left; op.padValue = _paddingVal;
    return out;
}

SliceLayer::SliceLayer(const int &batch, const int &height, const int &width, const int &channel, const int &start0, const int &step0,
                       const int &start1, const int &step1, const int &start2, const int &step2)
    : _start0(start0), _step0(step0), _start1(start1), _step1(step1), _start2(start2), _step2(step2)
{
    if (step0 <= 0 || step1 <= 0 || step2 <= 0 || start0 < 0 || start1 < 0 || start2 < 0) MSNH_THROW("slice: start must be >= 0 and step > 0");
    _type = LayerType::SLICE;
    _layerName = "Slice           ";
    _batch = batch; _height = height; _width = width; _channel = channel;
    if (start0 > channel - 1) MSNH_THROW("slice c start error");
    _outChannel = (channel - start0) / step0 + ((channel - start0) % step0 == 0 ? 0 : 1);
    if (start1 > height - 1) MSNH_THROW("slice h start error");
    _outHeight = (height - start1) / step1 + ((height - start1) % step1 == 0 ? 0 : 1);
    if (start2 > width - 1) MSNH_THROW("slice w start error");
    _outWidth = (width - start2) / step2 + ((width - start2) % step2 == 0 ? 0 : 1);
    _inputNum = width * height * channel;
    _outputNum = _outWidth * _outHeight * _outChannel;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("Slice                        %4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _width, _height, _channel, _outWidth, _outHeight,
                       _outChannel, 0.0);
}

int SliceLayer::lower(Plan &plan, int in, int layerIndex)
{
    in = plan.nhwcOf(in, layerIndex);
    const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
    if (ti.layout != PlanTensor::NHWC) MSNH_THROW("slice: the input must be an image tensor");
    const int out = plan.addTensor(ti.n, _outHeight, _outWidth, _outChannel, ti.dtype, "slice_out");
    PlanOp &op = plan.addOp(PlanOp::SLICE, in, -1, out, layerIndex, "slice");
    op.slice[0] = _start0; op.slice[1] = _step0; op.slice[2] = _start1; op.slice[3] = _step1; op.slice[4] = _start2; op.slice[5] = _step2;
    return out;
}

VariableOpLayer::VariableOpLayer(const int &batch, const int &width, const int &height, const int &channel, std::vector<int> &inputLayerIndexes,
                                 const VariableOpParams::VarOpType &varOpType, const float &constVal)
    : _inputLayerIndexes(inputLayerIndexes), _varOpType(varOpType), _constVal(constVal)
{
    const bool two = varOpType == VariableOpParams::VAR_OP_ADD || varOpType == VariableOpParams::VAR_OP_SUB || varOpType == VariableOpParams::VAR_OP_SUB_INV;
    const bool con = varOpType == VariableOpParams::VAR_OP_ADD_CONST || varOpType == VariableOpParams::VAR_OP_SUB_CONST ||
                     varOpType == VariableOpParams::VAR_OP_SUB_CONST_INV || varOpType == VariableOpParams::VAR_OP_MUL_CONST ||
                     varOpType == VariableOpParams::VAR_OP_DIV_CONST;
    if (!two && !con)
        MSNH_THROW("varop: " + VariableOpParams::getStrFromVarOpType(varOpType) + " is outside the convolutional path this build implements");
    if (two && (inputLayerIndexes.size() < 1 || inputLayerIndexes.size() > 2)) MSNH_THROW("varop: one or two input layers are needed");
    if (con && !inputLayerIndexes.empty()) MSNH_THROW("varop: constant forms take the previous layer as their input");
    if (varOpType == VariableOpParams::VAR_OP_DIV_CONST && constVal == 0.f) MSNH_THROW("varop: division by zero");
    _type = LayerType::VARIABLE_OP;
    _layerName = "VarOp           ";
    _batch = batch; _width = width; _height = height; _channel = channel;
    _outWidth = width; _outHeight = height; _outChannel = channel;
    _inputNum = width * height * channel; _outputNum = _inputNum;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = "VarOp Layer: " + VariableOpParams::getStrFromVarOpType(varOpType) + "\n";
}

void VariableOpLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    float a = 1.f, b = 0.f;
    switch (_varOpType)
    {
    case VariableOpParams::VAR_OP_ADD_CONST:     b = _constVal; break;
    case VariableOpParams::VAR_OP_SUB_CONST:     b = -_constVal; break;
    case VariableOpParams::VAR_OP_SUB_CONST_INV: a = -1.f; b = _constVal; break;
    case VariableOpParams::VAR_OP_MUL_CONST:     a = _constVal; break;
    case VariableOpParams::VAR_OP_DIV_CONST:     a = 1.f / _constVal; break;
    default: break;
    }
    scale.assign(static_cast<size_t>(_channel), a);
    shift.assign(static_cast<size_t>(_channel), b);
}

int VariableOpLayer::lower(Plan &plan, int in, int layerIndex)
{
    if (_inputLayerIndexes.empty())
    {
        in = plan.nhwcOf(in, layerIndex);
        const PlanTensor ti = plan.tensors[static_cast<size_t>(in)];
        if (ti.layout != PlanTensor::NHWC) MSNH_THROW("varop: the input must be an image tensor");
        const int out = plan.addTensor(ti.n, ti.h, ti.w, ti.c, ti.dtype, "varop_out");
        PlanOp &op = plan.addOp(PlanOp::AFFINE, in, -1, out, layerIndex, "varop_const");
        op.src = this;
        return out;
    }
    // one listed layer: A = previous layer, B = it; two: A, B = the listed layers (src/layers/MsnhVariableOpLayer.cpp:78-158)
    int a = in, b = plan.layerOut[static_cast<size_t>(_inputLayerIndexes[0])];
    if (_inputLayerIndexes.size() == 2) { a = b; b = plan.layerOut[static_cast<size_t>(_inputLayerIndexes[1])]; }
    a = plan.nhwcOf(a, layerIndex); b = plan.nhwcOf(b, layerIndex);
    const PlanTensor ta = plan.tensors[static_cast<size_t>(a)], tb = plan.tensors[static_cast<size_t>(b)];
    if (ta.layout != PlanTensor::NHWC || tb.layout != PlanTensor::NHWC || ta.h != tb.h || ta.w != tb.w || ta.c != tb.c)
        MSNH_THROW("varop: the two inputs must be image tensors of the same shape");
    if (_varOpType == VariableOpParams::VAR_OP_SUB_INV) std::swap(a, b);
    const int out = plan.addTensor(ta.n, ta.h, ta.w, ta.c, ta.dtype, "varop_out");
    PlanOp &op = plan.addOp(PlanOp::ADD, a, b, out, layerIndex, "varop");
    op.in1Sign = _varOpType == VariableOpParams::VAR_OP_ADD ? 1.f : -1.f;
    return out;
}

EmptyLayer::EmptyLayer(const int &batch, const int &width, const int &height, const int &channel)
{
    _type = LayerType::EMPTY;
    _layerName = "Empty           ";
    _batch = batch; _width = width; _height = height; _channel = channel;
    _outWidth = width; _outHeight = height; _outChannel = channel;
    _inputNum = width * height * channel;
    _outputNum = _inputNum;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _layerDetail = fmt("Empty Layer                  %4d x%4d x%4d -> %4d x%4d x%4d %5.3f BF\n", _width, _height, _channel, _outWidth, _outHeight,
                       _outChannel, 0.0);
}

int EmptyLayer::lower(Plan &, int in, int) { return in; }        // identity: the reference copies, the plan aliases

RouteLayer::RouteLayer(const int &batch, std::vector<int> &inputLayerIndexes, std::vector<int> &inputLayerOutputs, const int &groups,
                       const int &groupIndex, const int &addModel, const ActivationType &activation, const std::vector<float> &actParams)
    : _inputLayerIndexes(inputLayerIndexes), _inputLayerOutputs(inputLayerOutputs), _groups(groups), _groupIndex(groupIndex), _addModel(addModel)
{
    if (groups != 1) MSNH_THROW("route: groups are outside the convolutional path this build implements");
    if (addModel == 1 && inputLayerIndexes.size() < 2) MSNH_THROW("route layer error, add model must have at least 2 layers ");
    requireDeviceActivation(activation, "route");
    _type = LayerType::ROUTE;
    _layerName = "Route           ";
    _batch = batch;
    _activation = activation; _actParams = actParams;
    _layerDetail = "route ";
    int outputNum = 0;
    for (size_t i = 0; i < inputLayerIndexes.size(); ++i)
    {
        _layerDetail += fmt(" %d", inputLayerIndexes[i]);
        outputNum += inputLayerOutputs[i];
    }
    _layerDetail += "\n";
    if (addModel == 1) outputNum = inputLayerOutputs[0];
    _outputNum = outputNum;
    _inputNum = outputNum;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
}

int RouteLayer::lower(Plan &plan, int, int layerIndex)
{
    std::vector<int> srcs;
    for (int idx : _inputLayerIndexes) srcs.push_back(plan.nhwcOf(plan.layerOut[static_cast<size_t>(idx)], layerIndex));
    const PlanTensor first = plan.tensors[static_cast<size_t>(srcs[0])];
    int result;
    if (_addModel == 1)
    {
        // zero-filled output, then += every listed layer in list order (src/layers/MsnhRouteLayer.cpp:77-115); the last add takes the activation
        int acc = srcs[0];
        for (size_t i = 1; i < srcs.size(); ++i)
        {
            const PlanTensor t = plan.tensors[static_cast<size_t>(srcs[i])];
            if (t.h != first.h || t.w != first.w || t.c != first.c) MSNH_THROW("[route] layers height or width not equal.");
            const int out = plan.addTensor(first.n, first.h, first.w, first.c, first.dtype, "route_sum");
            PlanOp &op = plan.addOp(PlanOp::ADD, acc, srcs[i], out, layerIndex, "route_add");
            if (i + 1 == srcs.size()) { op.act = _activation; op.actParam = actParam(); }
            acc = out;
        }
        return acc;
    }
    if (srcs.size() == 1) result = srcs[0];                      // a single routed layer is an alias, not a copy
    else
    {
        int channels = 0;
        for (int s : srcs) channels += plan.tensors[static_cast<size_t>(s)].c;
        result = plan.addTensor(first.n, first.h, first.w, channels, first.dtype, "route_out");
        int off = 0;
        for (int s : srcs)
        {
            PlanOp &op = plan.addOp(PlanOp::COPY, s, -1, result, layerIndex, "route_copy");
            op.dstChanOffset = off;
            off += plan.tensors[static_cast<size_t>(s)].c;
        }
    }
    if (_activation != ActivationType::NONE)
    {
        const PlanTensor tr = plan.tensors[static_cast<size_t>(result)];
        const int out = plan.addTensor(tr.n, tr.h, tr.w, tr.c, tr.dtype, "route_act");
        PlanOp &op = plan.addOp(PlanOp::AFFINE, result, -1, out, layerIndex, "route_act");
        op.act = _activation; op.actParam = actParam();
        op.pureAct = true;
        op.src = this;
        result = out;
    }
    return result;
}

void RouteLayer::foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const
{
    scale.assign(static_cast<size_t>(_outChannel), 1.f);
    shift.assign(static_cast<size_t>(_outChannel), 0.f);
}

// ---- blocks -----------------------------------------------------------------------------------------------------------------------
BlockLayer::~BlockLayer()
{
    for (auto &chain : _chains)
        for (BaseLayer *l : chain) delete l;
}

std::vector<BaseLayer *> BlockLayer::buildChain(NetBuildParams &params, std::vector<BaseParams *> &nodes, const char *blockName, bool allowEmpty)
{
    std::vector<BaseLayer *> chain;
    try
    {
        for (size_t i = 0; i < nodes.size(); ++i)
        {
            BaseLayer *layer = nullptr;
            BaseParams *bp = nodes[i];
            if (bp->type == LayerType::CONVOLUTIONAL)
            {
                if (params.height == 0 || params.width == 0 || params.channels == 0) MSNH_THROW("Layer before convolutional layer must output image");
                ConvParams *p = static_cast<ConvParams *>(bp);
                layer = new ConvolutionalLayer(params.batch, 1, params.height, params.width, params.channels, p->filters, p->groups, p->kSizeX, p->kSizeY,
                                               p->strideX, p->strideY, p->dilationX, p->dilationY, p->paddingX, p->paddingY, p->activation, p->actParams,
                                               p->batchNorm, p->bnEps, p->useBias, 0, 0, 0, 0, p->antialiasing, nullptr, 0, 0);
            }
            else if (bp->type == LayerType::CONNECTED)
            {
                ConnectParams *p = static_cast<ConnectParams *>(bp);
                layer = new ConnectedLayer(params.batch, 1, params.inputNums, p->output, p->activation, p->actParams, p->batchNorm, p->bnEps, p->useBias);
            }
            else if (bp->type == LayerType::MAXPOOL)
            {
                MaxPoolParams *p = static_cast<MaxPoolParams *>(bp);
                layer = new MaxPoolLayer(params.batch, params.height, params.width, params.channels, p->kSizeX, p->kSizeY, p->strideX, p->strideY,
                                         p->paddingX, p->paddingY, p->maxPoolDepth, p->outChannels, p->ceilMode, 0);
            }
            else if (bp->type == LayerType::LOCAL_AVGPOOL)
            {
                LocalAvgPoolParams *p = static_cast<LocalAvgPoolParams *>(bp);
                layer = new LocalAvgPoolLayer(params.batch, params.height, params.width, params.channels, p->kSizeX, p->kSizeY, p->strideX, p->strideY,
                                              p->paddingX, p->paddingY, p->ceilMode, 0);
            }
            else if (bp->type == LayerType::BATCHNORM)
            {
                BatchNormParams *p = static_cast<BatchNormParams *>(bp);
                layer = new BatchNormLayer(params.batch, params.width, params.height, params.channels, p->activation, p->eps, p->actParams);
            }
            else if (allowEmpty && bp->type == LayerType::EMPTY)
            {
                layer = new EmptyLayer(params.batch, params.width, params.height, params.channels);
            }
            else
            {
                MSNH_THROW(std::string("layer type is not supported by [") + blockName + "]");
            }
            chain.push_back(layer);
            params.height = layer->getOutHeight();
            params.width = layer->getOutWidth();
            params.channels = layer->getOutChannel();
            params.inputNums = layer->getOutputNum();
            _maxOutputNum = std::max(_maxOutputNum, layer->getMaxOutputNum());
            _numWeights += layer->getNumWeights();
            _bFlops += layer->getBFlops();
            _layerDetail += layer->getLayerDetail();
            if (_type == LayerType::CONCAT_BLOCK) _layerDetail += "nweights  :" + std::to_string(layer->getNumWeights()) + "\n";
            layer->setIsBranchLayer(true);
            layer->setBranchFirst(i == 0);
            layer->setBranchLast(i + 1 == nodes.size());
        }
    }
    catch (...)
    {
        for (BaseLayer *l : chain) delete l;
        throw;
    }
    return chain;
}

void BlockLayer::loadAllWeigths(std::vector<float> &weights)
{
    if (weights.size() != _numWeights)
        MSNH_THROW(ExString::trim(_layerName) + " weights load err. needed : " + std::to_string(_numWeights) + " given : " + std::to_string(weights.size()));
    size_t ptr = 0;
    for (auto &chain : _chains)
        for (BaseLayer *l : chain)
        {
            const size_t n = l->getNumWeights();
            if (n == 0) continue;
            std::vector<float> part(weights.begin() + static_cast<long long>(ptr), weights.begin() + static_cast<long long>(ptr + n));
            l->loadAllWeigths(part);
            ptr += n;
        }
    _weightsLoaded = true;
}

void BlockLayer::weightLayout(std::vector<long long> &parts) const
{
    for (const auto &chain : _chains)
        for (const BaseLayer *l : chain) l->weightLayout(parts);
}

int BlockLayer::lowerChain(Plan &plan, const std::vector<BaseLayer *> &chain, int in, int layerIndex)
{
    int t = in;
    for (BaseLayer *l : chain) t = l->lower(plan, t, layerIndex);
    return t;
}

static int lowerAdd(Plan &plan, int a, int b, ActivationType act, float actParam, int layerIndex)
{
    const PlanTensor ta = plan.tensors[static_cast<size_t>(a)];
    const int out = plan.addTensor(ta.n, ta.h, ta.w, ta.c, ta.dtype, "add_out");
    PlanOp &op = plan.addOp(PlanOp::ADD, a, b, out, layerIndex, "add");
    op.act = act; op.actParam = actParam;
    return out;
}

static void checkBlockActivation(ActivationType act, const char *name)
{
    if (act == ActivationType::PRELU) MSNH_THROW(std::string("prelu activation is not supported by ") + name + " ");
    if (!Activations::deviceSupported(act)) MSNH_THROW(std::string(name) + ": activation is outside the convolutional path this build implements");
}

ResBlockLayer::ResBlockLayer(const int &batch, NetBuildParams &params, std::vector<BaseParams *> &baseParams, ActivationType &activation,
                             const std::vector<float> &actParams)
{
    checkBlockActivation(activation, "ResBlock");
    _type = LayerType::RES_BLOCK;
    _layerName = "ResBlock        ";
    _activation = activation; _actParams = actParams; _batch = batch;
    _width = params.width; _height = params.height; _channel = params.channels;
    _inputNum = params.width * params.height * params.channels;
    if (baseParams.empty()) MSNH_THROW("resblock has no layers");
    _layerDetail = "================================  ResBlock ================================\n";
    _chains.push_back(buildChain(params, baseParams, "ResBlockLayer", false));
    _outHeight = params.height; _outWidth = params.width; _outChannel = params.channels; _outputNum = params.inputNums;
    if (_outputNum != _inputNum) MSNH_THROW("resblock: the output of the block must have the size of its input");
    _layerDetail += "========================================================================\n";
}

int ResBlockLayer::lower(Plan &plan, int in, int layerIndex)
{
    const int f = lowerChain(plan, _chains[0], in, layerIndex);
    return lowerAdd(plan, f, in, _activation, actParam(), layerIndex);         // F(x) += x, then activation
}

Res2BlockLayer::Res2BlockLayer(const int &batch, NetBuildParams &params, std::vector<BaseParams *> &baseParams, std::vector<BaseParams *> &branchParams,
                               ActivationType &activation, const std::vector<float> &actParams)
{
    checkBlockActivation(activation, "Res2Block");
    _type = LayerType::RES_2_BLOCK;
    _layerName = "Res2Block       ";
    _activation = activation; _actParams = actParams; _batch = batch;
    _width = params.width; _height = params.height; _channel = params.channels;
    _inputNum = params.width * params.height * params.channels;
    if (baseParams.empty() || branchParams.empty()) MSNH_THROW("res2block needs a base and a branch");
    _layerDetail = "================================ Res2Block ================================\n";
    NetBuildParams branchBuild = params;
    _chains.push_back(buildChain(params, baseParams, "Res2BlockLayer", false));
    _chains.push_back(buildChain(branchBuild, branchParams, "Res2BlockLayer", false));
    if (params.height != branchBuild.height || params.width != branchBuild.width || params.channels != branchBuild.channels)
        MSNH_THROW("base's outputs size is not equal with branch's outputs size");
    _outHeight = params.height; _outWidth = params.width; _outChannel = params.channels; _outputNum = params.inputNums;
    _layerDetail += "========================================================================\n";
}

int Res2BlockLayer::lower(Plan &plan, int in, int layerIndex)
{
    const int base = lowerChain(plan, _chains[0], in, layerIndex);
    const int branch = lowerChain(plan, _chains[1], in, layerIndex);
    return lowerAdd(plan, branch, base, _activation, actParam(), layerIndex);  // branch += base, then activation
}

AddBlockLayer::AddBlockLayer(const int &batch, NetBuildParams &params, std::vector<std::vector<BaseParams *>> &branchParams, ActivationType &activation,
                             const std::vector<float> &actParams)
{
    checkBlockActivation(activation, "AddBlock");
    _type = LayerType::ADD_BLOCK;
    _layerName = "AddBlock        ";
    _activation = activation; _actParams = actParams; _batch = batch;
    _width = params.width; _height = params.height; _channel = params.channels;
    _inputNum = params.width * params.height * params.channels;
    if (branchParams.empty()) MSNH_THROW("addblock has no branch");
    if (branchParams.size() == 1 && activation != ActivationType::NONE)
        MSNH_THROW("addblock: a single branch with a block activation is outside the convolutional path this build implements");
    _layerDetail = "=============================== AddBlock ===============================\n";
    NetBuildParams last = params;
    for (size_t i = 0; i < branchParams.size(); ++i)
    {
        NetBuildParams bp = params;
        if (branchParams[i].empty()) MSNH_THROW("addblock: empty branch");
        _chains.push_back(buildChain(bp, branchParams[i], "AddBlockLayer", true));
        _layerDetail += "\n";
        if (i > 0 && (bp.height != last.height || bp.width != last.width || bp.channels != last.channels)) MSNH_THROW("branch's outputs size is not equal");
        last = bp;
    }
    params = last;
    _outHeight = last.height; _outWidth = last.width; _outChannel = last.channels; _outputNum = last.inputNums;
    _layerDetail += "========================================================================\n";
}

int AddBlockLayer::lower(Plan &plan, int in, int layerIndex)
{
    int acc = -1;
    for (size_t i = 0; i < _chains.size(); ++i)
    {
        const int y = lowerChain(plan, _chains[i], in, layerIndex);
        if (acc < 0) { acc = y; continue; }
        const bool lastBranch = i + 1 == _chains.size();
        acc = lowerAdd(plan, y, acc, lastBranch ? _activation : ActivationType::NONE, actParam(), layerIndex);      // b[i] += b[i-1]
    }
    return acc;
}

ConcatBlockLayer::ConcatBlockLayer(const int &batch, NetBuildParams &params, std::vector<std::vector<BaseParams *>> &branchParams,
                                   ActivationType &activation, const std::vector<float> &actParams)
{
    if (activation != ActivationType::NONE) MSNH_THROW("concatblock: a block activation is outside the convolutional path this build implements");
    _type = LayerType::CONCAT_BLOCK;
    _layerName = "ConcatBlock     ";
    _activation = activation; _actParams = actParams; _batch = batch;
    _width = params.width; _height = params.height; _channel = params.channels;
    _inputNum = params.width * params.height * params.channels;
    if (branchParams.empty()) MSNH_THROW("concatblock has no branch");
    _layerDetail = "=============================== ConcatBlock ===============================\n";
    int channels = 0;
    NetBuildParams last = params;
    for (size_t i = 0; i < branchParams.size(); ++i)
    {
        NetBuildParams bp = params;
        if (branchParams[i].empty()) MSNH_THROW("concatblock: empty branch");
        _chains.push_back(buildChain(bp, branchParams[i], "ConcatBlockLayer", true));
        _layerDetail += "\n";
        if (i > 0 && (bp.height != last.height || bp.width != last.width)) MSNH_THROW("branch's outputs size is not equal");
        channels += bp.channels;
        last = bp;
    }
    _outHeight = last.height; _outWidth = last.width; _outChannel = channels;
    _outputNum = _outHeight * _outWidth * _outChannel;
    params.height = _outHeight; params.width = _outWidth; params.channels = _outChannel; params.inputNums = _outputNum;
    _maxOutputNum = std::max(_maxOutputNum, static_cast<size_t>(_batch) * _outputNum);
    _layerDetail += "===========================================================================\n";
}

int ConcatBlockLayer::lower(Plan &plan, int in, int layerIndex)
{
    std::vector<int> outs;
    for (auto &chain : _chains) outs.push_back(lowerChain(plan, chain, in, layerIndex));
    const PlanTensor first = plan.tensors[static_cast<size_t>(outs[0])];
    const int out = plan.addTensor(first.n, first.h, first.w, _outChannel, first.dtype, "concat_out");
    int off = 0;
    for (int s : outs)
    {
        PlanOp &op = plan.addOp(PlanOp::COPY, s, -1, out, layerIndex, "concat_copy");
        op.dstChanOffset = off;
        off += plan.tensors[static_cast<size_t>(s)].c;
    }
    return out;
}

// ---- YOLO ------------------------------------------------------------------------------------------------------------------------------
YoloLayer::YoloLayer(const int &batch, const int &width, const int &height, const int &num, const int &orgWidth, const int &orgHeight,
                     const int &classNum, const std::vector<float> &anchors, const YoloType &yoloType)
    : anchors(anchors), _orgHeight(orgHeight), _orgWidth(orgWidth), _classNum(classNum), _yoloType(yoloType)
{
    _type = LayerType::YOLO;
    _layerName = "Yolo            ";
    _num = num; _batch = batch; _height = height; _width = width; _channel = num;
    _outWidth = width; _outHeight = height; _outChannel = num;
    _outputNum = height * width * num;
    _inputNum = _outputNum;
    _maxOutputNum = static_cast<size_t>(_batch) * _outputNum;
    _ratios = 1.f * orgHeight / _outHeight;          // height only, used for both axes (src/layers/MsnhYoloLayer.cpp:34)
    if (3 * (classNum + 4 + 1) != num) MSNH_THROW("class num error!");
    if (this->anchors.size() != 6) MSNH_THROW("[yolo] anchor num should be 6");
    if (yoloType != YoloType::YoloV3 && yoloType != YoloType::YoloV4 && yoloType != YoloType::YoloV5)
        MSNH_THROW("yolo: angle / gaussian variants are outside the convolutional path this build implements");
    _memReUse = 0;
    _layerDetail = "Yolo. class num : " + std::to_string(classNum) + "\n";
}

int YoloLayer::lower(Plan &plan, int in, int layerIndex)
{
    if (layerIndex == 0) MSNH_THROW("Yolo layer should not be 0 layer");
    // logits feeding the decode stay in float32: sigmoid / exp are evaluated on them exactly once
    const int p = plan.producerOf(in);
    if (p >= 0 && plan.ops[static_cast<size_t>(p)].kind == PlanOp::CONV && plan.consumerCount(in) == 0)
        plan.tensors[static_cast<size_t>(in)].dtype = MSNH_F32;
    const int out = plan.addTensor(_batch, _outHeight, _outWidth, _outChannel, MSNH_F32, "yolo_decoded", PlanTensor::FLAT);
    plan.tensors[static_cast<size_t>(out)].external = true;      // lives in Plan::yoloDecoded
    PlanOp &op = plan.addOp(PlanOp::YOLO_DECODE, in, -1, out, layerIndex, "yolo_decode");
    for (int i = 0; i < 6; ++i) op.anchors[static_cast<size_t>(i)] = anchors[static_cast<size_t>(i)];
    op.classes = _classNum;
    op.ratio = _ratios;
    op.yoloVersion = static_cast<int>(_yoloType) / 10;
    op.confThresh = 2.f;
    decodeOp = plan.ops.size() - 1;
    return out;
}

bool YoloOutLayer::keepClassScores = false;
int YoloOutLayer::deviceNms = 1;
static const size_t kRecordBytes = 12 * sizeof(float);     // one record of msnh_hip_yolo_nms
static const size_t kQuickRecords = 2048;                   // least number of records copied back with the counters, before their number is known

YoloOutLayer::YoloOutLayer(const int &batch, const int &orgWidth, const int &orgHeight, std::vector<int> &yoloIndexes, std::vector<YoloInfo> &yoloLayersInfo,
                           const float &confThresh, const float &nmsThresh, const int &useSotfNms, const YoloType &yoloType)
    : _confThresh(confThresh), _nmsThresh(nmsThresh), _useSoftNms(useSotfNms), _orgHeight(orgHeight), _orgWidth(orgWidth), _yoloType(yoloType),
      _yoloIndexes(yoloIndexes), _yoloLayersInfo(yoloLayersInfo)
{
    if (yoloType != YoloType::YoloV3 && yoloType != YoloType::YoloV4 && yoloType != YoloType::YoloV5) MSNH_THROW("yoloout: only yolov3 / yolov4 / yolov5 are implemented");
    _type = LayerType::YOLO_OUT;
    _layerName = "YoloOut         ";
    _batch = batch;
    _layerDetail = "YoloOut    ";
    for (size_t i = 0; i < yoloIndexes.size(); ++i)
    {
        _width += yoloLayersInfo[i].outWidth;
        _height += yoloLayersInfo[i].outHeight;
        _layerDetail += fmt(" %d", yoloIndexes[i]);
        _yoloAllInputNum += yoloLayersInfo[i].getOutputNum();
        if (yoloLayersInfo[i].outChannel != yoloLayersInfo[0].outChannel) MSNH_THROW("yoloout: heads disagree on the class count");
    }
    _channel = yoloLayersInfo[0].outChannel / 3;
    _pixels = _yoloAllInputNum / _channel;
    _layerDetail += "\n";
    _memReUse = 0;
}

int YoloOutLayer::lower(Plan &plan, int, int layerIndex)
{
    // claim the heads: give each its cell range inside an image's decoded rows and switch its candidate list on
    int cell = 0;
    for (size_t i = 0; i < _yoloIndexes.size(); ++i)
    {
        const int t = plan.layerOut[static_cast<size_t>(_yoloIndexes[i])];
        const int p = plan.producerOf(t);
        if (p < 0 || plan.ops[static_cast<size_t>(p)].kind != PlanOp::YOLO_DECODE) MSNH_THROW("yoloout layer error, not a yolo layer");
        PlanOp &op = plan.ops[static_cast<size_t>(p)];
        op.cellBase = cell;
        op.confThresh = _confThresh;
        cell += 3 * _yoloLayersInfo[i].outHeight * _yoloLayersInfo[i].outWidth;
    }
    plan.yoloCells = cell;
    plan.yoloClasses = _channel - 5;
    (void)layerIndex;
    return plan.addTensor(_batch, 1, 1, 0, MSNH_F32, "yoloout", PlanTensor::FLAT);
}

std::vector<YoloBox> YoloOutLayer::boxesFromRows(const float *rows, int count, const float *decodedOfImage) const
{
    return sortedCandidates(rows, count, decodedOfImage, _channel);
}

std::vector<YoloBox> YoloOutLayer::sortedCandidates(const float *rows, int count, const float *decodedOfImage, int channel)
{
    // Candidates arrive in arbitrary order; the reference scans cells in ascending order
    // (src/layers/MsnhYoloOutLayer.cpp:120-170), so restore that first.
    std::vector<int> order(static_cast<size_t>(count));
    for (int i = 0; i < count; ++i) order[static_cast<size_t>(i)] = i;
    std::sort(order.begin(), order.end(), [rows](int a, int b) { return rows[a * 8 + 7] < rows[b * 8 + 7]; });
    std::vector<YoloBox> boxes(static_cast<size_t>(count));
    std::vector<float> keys(static_cast<size_t>(count));
    for (int i = 0; i < count; ++i)
    {
        const float *r = rows + static_cast<size_t>(order[static_cast<size_t>(i)]) * 8;
        YoloBox &b = boxes[static_cast<size_t>(i)];
        b.xywhBox = Box::XYWHBox(r[0], r[1], r[2], r[3]);
        b.conf = r[4];
        b.bestClsConf = r[5];
        b.bestClsIdx = static_cast<int>(r[6]);
        if (decodedOfImage)
        {
            const float *row = decodedOfImage + static_cast<size_t>(r[7]) * channel;
            b.classesVal.assign(row + 5, row + channel);
        }
        keys[static_cast<size_t>(i)] = b.conf * b.bestClsConf;
    }
    // descending by objectness * best class score (:175-194)
    const std::vector<int> idx = ExVector::argsort(keys, true);
    std::vector<YoloBox> sorted(static_cast<size_t>(count));
    for (int i = 0; i < count; ++i) sorted[static_cast<size_t>(i)] = std::move(boxes[static_cast<size_t>(idx[static_cast<size_t>(i)])]);
    return sorted;
}

// Per-class greedy NMS exactly as the reference runs it (src/layers/MsnhYoloOutLayer.cpp:381-461): classes in
// first-appearance order, pick the highest objectness (first on ties), drop iou > thresh; a class with one
// box passes through.  NaN IoU (boxes with infinite extent) never suppresses, like there.
std::vector<YoloBox> YoloOutLayer::nms(const std::vector<YoloBox> &bboxes, const float &nmsThresh, const bool &useSoftNms, const float &sigma)
{
    std::vector<YoloBox> best;
    std::vector<int> classes;
    for (const YoloBox &b : bboxes)
        if (!ExVector::contains<int>(classes, b.bestClsIdx)) classes.push_back(b.bestClsIdx);
    std::vector<const YoloBox *> cur;
    for (int cls : classes)
    {
        cur.clear();
        for (const YoloBox &b : bboxes)
            if (b.bestClsIdx == cls) cur.push_back(&b);
        if (cur.size() == 1) { best.push_back(*cur[0]); continue; }
        while (!cur.empty())
        {
            size_t bi = 0;
            float bc = -FLT_MAX;
            for (size_t j = 0; j < cur.size(); ++j)
                if (cur[j]->conf > bc) { bi = j; bc = cur[j]->conf; }
            const YoloBox *top = cur[bi];
            best.push_back(*top);
            cur.erase(cur.begin() + static_cast<long long>(bi));
            size_t w = 0;
            for (size_t j = 0; j < cur.size(); ++j)
            {
                const float iou = Box::iou(cur[j]->xywhBox, top->xywhBox);
                bool drop;
                if (useSoftNms) drop = cur[j]->conf * std::exp(-(1.f * iou * iou / sigma)) <= 0;
                else drop = iou > nmsThresh;
                if (!drop) cur[w++] = cur[j];
            }
            cur.resize(w);
        }
    }
    return best;
}

// Same result as nms() for hard NMS, reorganised for speed: candidates of a class are visited in the order the
// greedy loop would pick them (objectness descending, earlier position first on ties) and each is kept unless a
// box kept before it overlaps it by more than the threshold -- that is exactly when the greedy loop would have
// erased it.  The kept boxes are held as structure-of-arrays so the IoU test runs 8 wide.
std::vector<YoloBox> YoloOutLayer::nmsSorted(const std::vector<YoloBox> &bboxes, float nmsThresh)
{
    std::vector<YoloBox> best;
    if (bboxes.empty()) return best;
    std::vector<std::vector<int>> members = groupByClass(bboxes);
    best.reserve(bboxes.size());
    for (std::vector<int> &m : members)
    {
        nmsClass(bboxes, m, nmsThresh);
        for (int j : m) best.push_back(bboxes[static_cast<size_t>(j)]);
    }
    return best;
}

// indices of the candidates of each class, classes in first-appearance order
std::vector<std::vector<int>> YoloOutLayer::groupByClass(const std::vector<YoloBox> &bboxes)
{
    int maxCls = 0;
    for (const YoloBox &b : bboxes) maxCls = std::max(maxCls, b.bestClsIdx);
    std::vector<int> slotOf(static_cast<size_t>(maxCls) + 1, -1);
    std::vector<std::vector<int>> members;
    for (size_t i = 0; i < bboxes.size(); ++i)
    {
        const int c = bboxes[i].bestClsIdx;
        if (c < 0) MSNH_THROW("negative class index");
        if (slotOf[static_cast<size_t>(c)] < 0)
        {
            slotOf[static_cast<size_t>(c)] = static_cast<int>(members.size());
            members.emplace_back();
        }
        members[static_cast<size_t>(slotOf[static_cast<size_t>(c)])].push_back(static_cast<int>(i));
    }
    return members;
}

// greedy NMS inside one class: on return m holds the kept candidates in pick order
void YoloOutLayer::nmsClass(const std::vector<YoloBox> &bboxes, std::vector<int> &m, float nmsThresh)
{
    if (m.size() <= 1) return;
    std::stable_sort(m.begin(), m.end(), [&bboxes](int a, int b) { return bboxes[static_cast<size_t>(a)].conf > bboxes[static_cast<size_t>(b)].conf; });
    std::vector<float> kx1, ky1, kx2, ky2, karea;
    size_t w = 0;
    for (int j : m)
    {
        const Box::XYWHBox &q = bboxes[static_cast<size_t>(j)].xywhBox;
        const float jx1 = q.x - q.w / 2.f, jx2 = q.x + q.w / 2.f, jy1 = q.y - q.h / 2.f, jy2 = q.y + q.h / 2.f;
        const float jarea = (jx2 - jx1 + 1) * (jy2 - jy1 + 1);
        const size_t nk = kx1.size();
        int hit = 0;
        // the kept boxes are tested in blocks: most candidates of a crowded class are erased by one of the first
        // (highest-objectness) kept boxes, and any hit decides
        for (size_t k0 = 0; k0 < nk && !hit; k0 += 64)
        {
            const size_t k1 = std::min(nk, k0 + 64);
#pragma omp simd reduction(| : hit)
            for (size_t k = k0; k < k1; ++k)
            {
                // Box::iou(candidate j, kept k) with std::min / std::max spelled out
                const float ix2 = (kx2[k] < jx2) ? kx2[k] : jx2;
                const float ix1 = (jx1 < kx1[k]) ? kx1[k] : jx1;
                const float iy2 = (ky2[k] < jy2) ? ky2[k] : jy2;
                const float iy1 = (jy1 < ky1[k]) ? ky1[k] : jy1;
                const float iw = ix2 - ix1 + 1;
                const float ih = iy2 - iy1 + 1;
                const float inter = (iw < 0 ? 0 : iw) * (ih < 0 ? 0 : ih);
                const float iou = 1.f * inter / (jarea + karea[k] - inter);
                hit |= (iou > nmsThresh) ? 1 : 0;
            }
        }
        if (hit) continue;
        m[w++] = j;
        kx1.push_back(jx1); ky1.push_back(jy1); kx2.push_back(jx2); ky2.push_back(jy2); karea.push_back(jarea);
    }
    m.resize(w);
}

// Undo the letterbox (square padding + uniform scale): the padding is on the short side of the original image.
YoloBox YoloOutLayer::bboxResize2Org(YoloBox &box, const Point2I &currentShape, const Point2I &orgShape)
{
    const int orgW = orgShape.x, orgH = orgShape.y, curW = currentShape.x, curH = currentShape.y;
    if (orgW > orgH)
    {
        const float ratio = 1.0f * curW / orgW;
        const int padUp = static_cast<int>((curH - orgH * ratio) / 2);
        box.xywhBox.x = box.xywhBox.x / ratio;
        box.xywhBox.w = box.xywhBox.w / ratio;
        box.xywhBox.y = (box.xywhBox.y - padUp) / ratio;
        box.xywhBox.h = box.xywhBox.h / ratio;
    }
    else
    {
        const float ratio = 1.0f * curH / orgH;
        const int padLeft = static_cast<int>((curW - orgW * ratio) / 2);
        box.xywhBox.x = (box.xywhBox.x - padLeft) / ratio;
        box.xywhBox.w = box.xywhBox.w / ratio;
        box.xywhBox.y = box.xywhBox.y / ratio;
        box.xywhBox.h = box.xywhBox.h / ratio;
    }
    return box;
}

// Undo a plain resize that did not keep the aspect ratio.
YoloBox YoloOutLayer::bboxResize2OrgNoPad(YoloBox &box, const Point2I &currentShape, const Point2I &orgShape)
{
    const float ratioW = 1.0f * currentShape.x / orgShape.x;
    const float ratioH = 1.0f * currentShape.y / orgShape.y;
    box.xywhBox.x = box.xywhBox.x / ratioW;
    box.xywhBox.w = box.xywhBox.w / ratioW;
    box.xywhBox.y = box.xywhBox.y / ratioH;
    box.xywhBox.h = box.xywhBox.h / ratioH;
    return box;
}

void YoloOutLayer::enqueueGather(msnh_stream_t s)
{
    if (plan == nullptr) MSNH_THROW("YoloOut: layer is not part of a planned network");
    Plan &pl = *plan;
    if (pl.sparseYolo) return;          // the heads' candidate-only decode already wrote the compact rows
    MSNH_DEV(msnh_hip_yolo_gather(_batch, _channel - 5, pl.yoloDecoded.as<float>(), static_cast<long long>(pl.yoloCells) * _channel,
                                  pl.yoloCandIdx.as<int>(), pl.yoloCells, pl.yoloCandCnt.as<int>(), pl.yoloRows.as<float>(), s));
}

// Everything a slot needs, at its full size, before the slot is first used.  An allocation or a free of device or pinned memory
// waits for the whole device: in the middle of a run, with other instances' forwards in flight, one such call stalls them all
// for tens of milliseconds.  Both slots are prepared with the first forward (later calls find everything in place).
void YoloOutLayer::prepareSlot(Slot &sl, bool deviceNmsBuffers)
{
    Plan &pl = *plan;
    const size_t cells = static_cast<size_t>(pl.yoloCells);
    const size_t cntBytes = sizeof(int) * static_cast<size_t>(_batch);
    const size_t rowBytes = sizeof(float) * 8 * cells * static_cast<size_t>(_batch);
    sl.cnt.reserve(cntBytes);
    sl.rows.reserve(rowBytes);
    if (sl.event == nullptr) MSNH_DEV(msnh_hip_event_create(&sl.event));
    if (keepClassScores) return;
    if (sl.ready == nullptr) MSNH_DEV(msnh_hip_event_create(&sl.ready));
    if (sl.devCnt.bytes() < cntBytes) sl.devCnt.alloc(cntBytes);
    if (sl.devRows.bytes() < rowBytes) sl.devRows.alloc(rowBytes);
    if (!deviceNmsBuffers) return;
    const size_t keptCntBytes = sizeof(int) * (1 + static_cast<size_t>(_batch));
    const size_t keptCap = cells * static_cast<size_t>(_batch);
    if (sl.devKeptCnt.bytes() < keptCntBytes) sl.devKeptCnt.alloc(keptCntBytes);
    if (sl.devKept.bytes() < keptCap * kRecordBytes) sl.devKept.alloc(keptCap * kRecordBytes);
    sl.keptCnt.reserve(keptCntBytes);
    sl.kept.reserve(keptCap * kRecordBytes);
    const size_t wsBytes = msnh_hip_yolo_nms_pair_workspace_bytes(_batch, _channel - 5, pl.yoloCells);
    if (sl.devNmsWs.bytes() < wsBytes) sl.devNmsWs.alloc(wsBytes);
}

void YoloOutLayer::enqueueCopyBack(msnh_stream_t s, int slot)
{
    Plan &pl = *plan;
    Slot &sl = _slots[slot & 1];
    if (sl.pending) MSNH_THROW("YoloOut: the results of the previous forward in this slot were not fetched");
    sl.onDevice = false;
    const size_t cells = static_cast<size_t>(pl.yoloCells);
    const bool mayUseDevice = deviceNms != 0 && !_useSoftNms && !keepClassScores;
    prepareSlot(_slots[0], mayUseDevice);
    prepareSlot(_slots[1], mayUseDevice);
    const size_t cntBytes = sizeof(int) * static_cast<size_t>(_batch);
    const size_t rowBytes = sizeof(float) * 8 * cells * static_cast<size_t>(_batch);
    if (keepClassScores)
    {
        // the decoded tensor is too large to snapshot: everything leaves on the forward's own stream
        MSNH_DEV(msnh_hip_memcpy_d2h(sl.cnt.ptr(), pl.yoloCandCnt.ptr(), cntBytes, s));
        MSNH_DEV(msnh_hip_memcpy_d2h(sl.rows.ptr(), pl.yoloRows.ptr(), rowBytes, s));
        const size_t bytes = sizeof(float) * cells * static_cast<size_t>(_channel) * static_cast<size_t>(_batch);
        sl.decoded.reserve(bytes);
        MSNH_DEV(msnh_hip_memcpy_d2h(sl.decoded.ptr(), pl.yoloDecoded.ptr(), bytes, s));
        MSNH_DEV(msnh_hip_event_record(sl.event, s));
        sl.pending = true;
        sl.rowsCopied = cells;
        return;
    }
    // Snapshot on the device (microseconds), then cross PCIe on a second stream: the next forward does not wait for
    // the copy (several MiB: every cell has a row slot, the count is only known on the device).
    // copyOnForwardStream (the instances of a NetGroup): everything below goes onto the forward's own stream.  A process has four
    // hardware queues; three instances with a copy stream each are six busy streams, and a copy stream that shares a queue with
    // another instance's forward waits behind that forward's kernels (measured: 4150-4750 images/s depending on nothing but the
    // order in which the streams were created).  On its own stream the copy sits between two forwards of the instance, and the
    // other instances fill the gap.
    if (!copyOnForwardStream && _copyStream == nullptr) MSNH_DEV(msnh_hip_stream_create(&_copyStream));
    const msnh_stream_t cs = copyOnForwardStream ? s : _copyStream;
    MSNH_DEV(msnh_hip_memcpy_d2d(sl.devCnt.ptr(), pl.yoloCandCnt.ptr(), cntBytes, s));
    MSNH_DEV(msnh_hip_memcpy_d2d(sl.devRows.ptr(), pl.yoloRows.ptr(), rowBytes, s));
    MSNH_DEV(msnh_hip_event_record(sl.ready, s));
    if (!copyOnForwardStream) MSNH_DEV(msnh_hip_stream_wait_event(cs, sl.ready));
    MSNH_DEV(msnh_hip_memcpy_d2h(sl.cnt.ptr(), sl.devCnt.ptr(), cntBytes, cs));
    // auto: few candidates (real detections) -> the device; thousands per image -> the device too unless a second forward is in flight
    // (the host's sort + NMS then runs beside that forward and costs the device nothing, whereas the device NMS takes about 0.1 ms of
    // device time per batch from it) and the host stage has kept up with the device so far
    const bool pipelined = _slots[(slot ^ 1) & 1].pending;
    const bool mid = _lastMaxCandidates > kDeviceNmsFew && _lastMaxCandidates <= kDeviceNmsCandidates;
    sl.trial = deviceNms == 1 && !_useSoftNms && mid && pipelined && !_hostBound && _trialLeft > 0 && !copyOnForwardStream;
    if (sl.trial) --_trialLeft;
    // (on the forward's own stream the device NMS would sit in front of the instance's next forward: the instances of a group keep
    //  thousands of candidates on the host, which works beside the other instances' forwards)
    const bool autoDevice = _lastMaxCandidates <= kDeviceNmsFew || (mid && !copyOnForwardStream && (!pipelined || _hostBound || sl.trial));
    sl.onDevice = !_useSoftNms && (deviceNms == 2 || (deviceNms == 1 && autoDevice));
    if (sl.onDevice)
    {
        // NMS on the snapshot, on the copy stream: it overlaps the next forward, and what crosses PCIe is the kept boxes.  The records
        // leave with the counters, as many as the previous result had and half as many again: a copy asked for in finish() would
        // queue behind whatever the device runs by then (the next forward), and the host would wait for that instead of working
        // beside it.  finish() fetches the rest only if there are more.
        const size_t keptCntBytes = sizeof(int) * (1 + static_cast<size_t>(_batch));
        const size_t keptCap = cells * static_cast<size_t>(_batch);
        sl.quick = std::min(keptCap, std::max(kQuickRecords, _lastKept + _lastKept / 2 + 1024));
        MSNH_DEV(msnh_hip_fill_zero(sl.devKeptCnt.ptr(), keptCntBytes, cs));
        const size_t wsBytes = msnh_hip_yolo_nms_pair_workspace_bytes(_batch, _channel - 5, pl.yoloCells);
        MSNH_DEV(msnh_hip_yolo_nms(_batch, _channel - 5, sl.devRows.as<float>(), pl.yoloCells, sl.devCnt.as<int>(), _nmsThresh, sl.devKept.as<float>(),
                                   static_cast<int>(keptCap), sl.devKeptCnt.as<int>(), sl.devNmsWs.ptr(), wsBytes, cs));
        MSNH_DEV(msnh_hip_memcpy_d2h(sl.keptCnt.ptr(), sl.devKeptCnt.ptr(), keptCntBytes, cs));
        MSNH_DEV(msnh_hip_memcpy_d2h(sl.kept.ptr(), sl.devKept.ptr(), sl.quick * kRecordBytes, cs));
    }
    else
    {
        // Every cell has a row slot and the count is known only on the device; all slots are several MiB and their copy sits
        // between the end of a forward and the host stage of its batch.  So only a prefix of every image's slots is copied ahead
        // of time, sized from the previous result (half as much again, + 1024); finish() fetches what an image has beyond it.
        size_t guess = _lastMaxCandidates > 0 ? static_cast<size_t>(_lastMaxCandidates) + static_cast<size_t>(_lastMaxCandidates) / 2 + 1024 : cells;
        if (const char *forced = std::getenv("MSNH_YOLO_ROWS_PREFIX")) guess = static_cast<size_t>(std::max(1L, std::atol(forced)));    // (tests)
        sl.rowsCopied = std::min(guess, cells);
        if (sl.rowsCopied == cells)
            MSNH_DEV(msnh_hip_memcpy_d2h(sl.rows.ptr(), sl.devRows.ptr(), rowBytes, cs));
        else
            for (int b = 0; b < _batch; ++b)
            {
                const size_t off = static_cast<size_t>(b) * cells * 8;
                MSNH_DEV(msnh_hip_memcpy_d2h(sl.rows.as<float>() + off, sl.devRows.as<float>() + off, sizeof(float) * 8 * sl.rowsCopied, cs));
            }
    }
    MSNH_DEV(msnh_hip_event_record(sl.event, cs));
    sl.pending = true;
}

// Boxes of one image from the device's NMS records, in the reference's output order: classes by the first appearance in
// the score-sorted candidate list (= by their best-scoring candidate), inside a class in pick order.
std::vector<YoloBox> YoloOutLayer::boxesFromKept(std::vector<const float *> &records) const
{
    std::sort(records.begin(), records.end(), [](const float *a, const float *b) {
        if (a[8] != b[8]) return a[8] > b[8];
        if (a[9] != b[9]) return a[9] < b[9];
        return a[10] < b[10];
    });
    std::vector<YoloBox> out(records.size());
    for (size_t i = 0; i < records.size(); ++i)
    {
        const float *r = records[i];
        YoloBox &b = out[i];
        b.xywhBox = Box::XYWHBox(r[0], r[1], r[2], r[3]);
        b.conf = r[4];
        b.bestClsConf = r[5];
        b.bestClsIdx = static_cast<int>(r[6]);
    }
    return out;
}

// Time between consecutive results while two batches are in flight: a moving mean for the host placement, a plain mean over a
// device trial (its first four results still carry the change-over).  At the end of a trial the faster placement stays; a
// trial that lost is not repeated for a thousand batches.
void YoloOutLayer::noteResult(const Slot &sl, bool pipelined)
{
    const std::chrono::steady_clock::time_point now = std::chrono::steady_clock::now();
    const bool usable = _haveLastFinish && pipelined;
    const double ms = usable ? std::chrono::duration<double, std::milli>(now - _lastFinish).count() : 0.0;
    if (!sl.onDevice)
    {
        if (usable && _lastFinishHost) _hostInterval = _hostInterval > 0.0 ? _hostInterval + (ms - _hostInterval) / 8.0 : ms;
    }
    else if (sl.trial)
    {
        ++_trialSeen;
        if (usable && _trialSeen > 4) { _trialSum += ms; ++_trialSamples; }
        if (_trialSeen == kTrialBatches)
        {
            const bool faster = _trialSamples >= kTrialBatches / 2 && _trialSum / _trialSamples < 0.97 * _hostInterval;
            if (std::getenv("MSNH_DEBUG_TIMING"))
                std::fprintf(stderr, "yoloout placement trial: device %.3f ms (%d results), host %.3f ms between results -> %s\n",
                             _trialSamples ? _trialSum / _trialSamples : 0.0, _trialSamples, _hostInterval, faster ? "device" : "host");
            _hostBound = faster;
            _hostBoundRuns = faster ? 0 : -1000;
            _trialSeen = 0;
            _trialLeft = 0;
        }
    }
    _lastFinish = now;
    _haveLastFinish = true;
    _lastFinishHost = !sl.onDevice;
}

void YoloOutLayer::finish(int slot)
{
    Slot &sl = _slots[slot & 1];
    if (!sl.pending) MSNH_THROW("YoloOut: nothing to fetch");
    auto dbg0 = TimeUtil::startRecord();
    MSNH_DEV(msnh_hip_event_sync(sl.event));
    const float dbgWait = TimeUtil::getElapsedTime(dbg0);
    sl.pending = false;
    _lastSlot = slot & 1;
    lastOnDevice = sl.onDevice;
    noteResult(sl, _slots[(slot ^ 1) & 1].pending);
    const int cells = plan->yoloCells;
    const int per = _channel;
    const int *cnt = sl.cnt.as<int>();
    _lastMaxCandidates = 0;
    for (int b = 0; b < _batch; ++b) _lastMaxCandidates = std::max(_lastMaxCandidates, std::min(cnt[b], cells));
    if (sl.onDevice)
    {
        const int *keptCnt = sl.keptCnt.as<int>();
        const size_t total = static_cast<size_t>(keptCnt[0]);
        // (its own stream: the copy stream may already hold the next forward's work)
        if (_fetchStream == nullptr) MSNH_DEV(msnh_hip_stream_create(&_fetchStream));
        _lastKept = total;
        const size_t quick = sl.quick;
        if (total > quick)
        {
            PinnedBuffer &rest = sl.rows;                                  // the host path's buffer doubles as the overflow area
            rest.reserve((total - quick) * kRecordBytes);
            MSNH_DEV(msnh_hip_memcpy_d2h(rest.ptr(), sl.devKept.as<char>() + quick * kRecordBytes, (total - quick) * kRecordBytes, _fetchStream));
            MSNH_DEV(msnh_hip_stream_sync(_fetchStream));
        }
        std::vector<std::vector<const float *>> perImage(static_cast<size_t>(_batch));
        for (size_t i = 0; i < total; ++i)
        {
            const float *r = i < quick ? sl.kept.as<float>() + i * 12 : sl.rows.as<float>() + (i - quick) * 12;
            const int b = static_cast<int>(r[11]);
            if (b < 0 || b >= _batch) MSNH_THROW("YoloOut: device NMS record names image " + std::to_string(b));
            perImage[static_cast<size_t>(b)].push_back(r);
        }
        batchHasBox.assign(static_cast<size_t>(_batch), false);
        finalOut.assign(static_cast<size_t>(_batch), std::vector<YoloBox>());
        TaskPool::instance().parallelFor(_batch, [&](int b) {
            if (keptCnt[1 + b] == 0) finalOut[static_cast<size_t>(b)] = boxesFromKept(perImage[static_cast<size_t>(b)]);
        });
        std::vector<float> hostRows;
        for (int b = 0; b < _batch; ++b)
        {
            batchHasBox[static_cast<size_t>(b)] = cnt[b] > 0;
            if (keptCnt[1 + b] == 0) continue;
            // the device left this image to the host (a class with very many candidates, or NaN scores): the snapshot still holds its rows
            const int n = std::min(cnt[b], cells);
            hostRows.resize(static_cast<size_t>(n) * 8);
            MSNH_DEV(msnh_hip_memcpy_d2h(hostRows.data(), sl.devRows.as<float>() + static_cast<size_t>(b) * cells * 8, hostRows.size() * sizeof(float), _fetchStream));
            MSNH_DEV(msnh_hip_stream_sync(_fetchStream));
            finalOut[static_cast<size_t>(b)] = nmsSorted(boxesFromRows(hostRows.data(), n, nullptr), _nmsThresh);
        }
        if (std::getenv("MSNH_DEBUG_TIMING")) std::fprintf(stderr, "yoloout finish (device NMS, %zu boxes): wait %.3f ms, host %.3f ms\n", total, dbgWait, TimeUtil::getElapsedTime(dbg0) - dbgWait);
        return;
    }
    {
        // rows beyond the prefix that was copied ahead of time (the device snapshot of this slot is still intact)
        bool more = false;
        for (int b = 0; b < _batch; ++b)
        {
            const size_t n = static_cast<size_t>(std::min(cnt[b], cells));
            if (n <= sl.rowsCopied) continue;
            if (_fetchStream == nullptr) MSNH_DEV(msnh_hip_stream_create(&_fetchStream));
            const size_t off = (static_cast<size_t>(b) * static_cast<size_t>(cells) + sl.rowsCopied) * 8;
            MSNH_DEV(msnh_hip_memcpy_d2h(sl.rows.as<float>() + off, sl.devRows.as<float>() + off, sizeof(float) * 8 * (n - sl.rowsCopied), _fetchStream));
            more = true;
        }
        if (more) MSNH_DEV(msnh_hip_stream_sync(_fetchStream));
    }
    const float *decodedHost = keepClassScores ? sl.decoded.as<float>() : nullptr;
    batchHasBox.assign(static_cast<size_t>(_batch), false);
    finalOut.assign(static_cast<size_t>(_batch), std::vector<YoloBox>());
    // three flat parallel phases: candidates per image; NMS per (image, class) -- the classes of an image are
    // independent, and a batch has far fewer images than the host has cores; concatenation per image
    std::vector<std::vector<YoloBox>> cand(static_cast<size_t>(_batch));
    std::vector<std::vector<std::vector<int>>> groups(static_cast<size_t>(_batch));
    TaskPool &pool = TaskPool::instance();
    pool.parallelFor(_batch, [&](int b) {
        const int n = std::min(cnt[b], cells);
        const float *dec = decodedHost ? decodedHost + static_cast<size_t>(b) * cells * per : nullptr;
        cand[static_cast<size_t>(b)] = boxesFromRows(sl.rows.as<float>() + static_cast<size_t>(b) * cells * 8, n, dec);
        if (_useSoftNms) finalOut[static_cast<size_t>(b)] = nms(cand[static_cast<size_t>(b)], _nmsThresh, true);
        else groups[static_cast<size_t>(b)] = groupByClass(cand[static_cast<size_t>(b)]);
    });
    const double dbgA = TimeUtil::getElapsedTime(dbg0);
    double dbgB = dbgA;
    if (!_useSoftNms)
    {
        std::vector<std::pair<int, int>> tasks;
        for (int b = 0; b < _batch; ++b)
            for (size_t g = 0; g < groups[static_cast<size_t>(b)].size(); ++g) tasks.emplace_back(b, static_cast<int>(g));
        // largest classes first, one task at a time: a crowded class costs as much as all the small ones together
        std::stable_sort(tasks.begin(), tasks.end(), [&groups](const std::pair<int, int> &x, const std::pair<int, int> &y) {
            return groups[static_cast<size_t>(x.first)][static_cast<size_t>(x.second)].size() > groups[static_cast<size_t>(y.first)][static_cast<size_t>(y.second)].size();
        });
        const int nTasks = static_cast<int>(tasks.size());
        pool.parallelFor(nTasks, [&](int t) {
            const size_t b = static_cast<size_t>(tasks[static_cast<size_t>(t)].first);
            nmsClass(cand[b], groups[b][static_cast<size_t>(tasks[static_cast<size_t>(t)].second)], _nmsThresh);
        });
        dbgB = TimeUtil::getElapsedTime(dbg0);
        pool.parallelFor(_batch, [&](int b) {
            std::vector<YoloBox> &out = finalOut[static_cast<size_t>(b)];
            for (const std::vector<int> &m : groups[static_cast<size_t>(b)])
                for (int j : m) out.push_back(cand[static_cast<size_t>(b)][static_cast<size_t>(j)]);
        });
    }
    for (int b = 0; b < _batch; ++b) batchHasBox[static_cast<size_t>(b)] = cnt[b] > 0;
    {
        // did the device make the host wait?  If it has not for eight batches in a row, the host stage may be what bounds the
        // pipeline: the automatic mode then tries the device for kTrialBatches batches (noteResult() compares the two)
        const double stage = TimeUtil::getElapsedTime(dbg0) - dbgWait;
        if (_lastMaxCandidates <= kDeviceNmsFew) { _hostBoundRuns = 0; _hostBound = false; }
        else if (dbgWait < 0.05 * stage)
        {
            if (++_hostBoundRuns >= 8 && _trialLeft == 0 && _trialSeen == 0 && _hostInterval > 0.0) { _trialLeft = kTrialBatches; _trialSum = 0.0; _trialSamples = 0; }
        }
        else if (_hostBoundRuns > 0) _hostBoundRuns = 0;
    }
    if (std::getenv("MSNH_DEBUG_TIMING"))
        std::fprintf(stderr, "yoloout finish: wait %.3f ms, host %.3f ms (candidates %.3f, suppression %.3f, output %.3f)\n", dbgWait,
                     TimeUtil::getElapsedTime(dbg0) - dbgWait, dbgA - dbgWait, dbgB - dbgA, TimeUtil::getElapsedTime(dbg0) - dbgB);
}

std::vector<float> YoloOutLayer::lastCandidateRows(int image) const
{
    if (_lastSlot < 0) MSNH_THROW("YoloOut: no result was fetched yet");
    if (image < 0 || image >= _batch) MSNH_THROW("YoloOut: no such image in the batch");
    const Slot &sl = _slots[_lastSlot];
    if (sl.onDevice) MSNH_THROW("YoloOut: the last result was suppressed on the device, its candidate rows did not come to the host (device NMS mode 0 keeps them)");
    const size_t cells = static_cast<size_t>(plan->yoloCells);
    const size_t n = static_cast<size_t>(std::min(sl.cnt.as<int>()[image], plan->yoloCells));
    const float *rows = sl.rows.as<float>() + static_cast<size_t>(image) * cells * 8;
    return std::vector<float>(rows, rows + n * 8);
}

std::string YoloOutLayer::placementDetail() const
{
    if (_lastSlot < 0) return "YoloOut NMS     : no result yet\n";
    std::string d = std::string("YoloOut NMS     : last result on the ") + (lastOnDevice ? "device" : "host") + ", mode " +
                    (_useSoftNms ? "soft (host)" : (deviceNms == 0 ? "host" : (deviceNms == 2 ? "device" : "auto"))) + ", " + std::to_string(_lastMaxCandidates) +
                    " candidates in the fullest image";
    if (deviceNms == 1 && !_useSoftNms)
    {
        d += fmt("; host stage between results %.3f ms", _hostInterval);
        if (_trialLeft > 0 || _trialSeen > 0) d += fmt("; device trial running (%d of %d batches seen)", _trialSeen, kTrialBatches);
        else if (_hostBound) d += "; a device trial won: thousands of candidates stay on the device";
        else if (_hostBoundRuns < 0) d += "; a device trial lost: not repeated for a thousand batches";
    }
    return d + "\n";
}

void YoloOutLayer::forwardGPU(NetworkState &netState)
{
    enqueueGather(netState.stream);
    enqueueCopyBack(netState.stream, 0);
    finish(0);
}

YoloOutLayer::~YoloOutLayer()
{
    for (Slot &sl : _slots)
    {
        if (sl.event) msnh_hip_event_destroy(sl.event);
        if (sl.ready) msnh_hip_event_destroy(sl.ready);
    }
    if (_copyStream) msnh_hip_stream_destroy(_copyStream);
    if (_fetchStream) msnh_hip_stream_destroy(_fetchStream);
}
}
