// The concrete layer classes of the convolutional path.  Constructor parameter lists are the reference's
// (so code that builds layers by hand keeps compiling); see the per-class citations.
#pragma once
#include "Msnhnet/io/MsnhParser.h"
#include "Msnhnet/layers/MsnhBaseLayer.h"
#include "Msnhnet/layers/MsnhYoloDef.h"

namespace Msnhnet
{
class NetBuildParams
{
public:
    int batch = 0, inputNums = 0, height = 0, width = 0, channels = 0;
};

// src/layers/MsnhConvolutionalLayer.cpp:5-319 (ctor, shapes, weight count), :1186-1434 (weights)
class MsnhNet_API ConvolutionalLayer : public BaseLayer
{
public:
    ConvolutionalLayer(const int &batch, const int &steps, const int &height, const int &width, const int &channel, const int &num,
                       const int &groups, const int &kSizeX, const int &kSizeY, const int &strideX, const int &strideY,
                       const int &dilationX, const int &dilationY, const int &paddingX, const int &paddingY,
                       ActivationType activation, const std::vector<float> &actParams, const int &batchNorm, const float &bnEps,
                       const int &useBias, const int &binary, const int &xnor, const int &useBinOutput, const int &groupIndex,
                       const int &antialiasing, ConvolutionalLayer *const &shareLayer, const int &assistedExcitation, const int &deform);
    int convOutHeight() const;
    int convOutWidth() const;
    void loadAllWeigths(std::vector<float> &weights) override;
    void weightLayout(std::vector<long long> &parts) const override;
    int lower(Plan &plan, int in, int layerIndex) override;
    const std::vector<float> &kernelWeights() const override { return _weights; }
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;

    int getKSizeX() const { return _kSizeX; }
    int getKSizeY() const { return _kSizeY; }
    int getStride() const { return _strideX; }
    int getStrideX() const { return _strideX; }
    int getStrideY() const { return _strideY; }
    int getPaddingX() const { return _paddingX; }
    int getPaddingY() const { return _paddingY; }
    int getDilationX() const { return _dilationX; }
    int getDilationY() const { return _dilationY; }
    int getGroups() const { return _groups; }
    int getBatchNorm() const { return _batchNorm; }
    int getUseBias() const { return _useBias; }
    int getNBiases() const { return _nBiases; }
    int getNWeights() const { return _nWeights; }
    int getNScales() const { return _nScales; }
    int getNRollMean() const { return _nRollMean; }
    int getNRollVariance() const { return _nRollVariance; }

private:
    int _groups = 1, _kSizeX = 1, _kSizeY = 1, _strideX = 1, _strideY = 1, _dilationX = 1, _dilationY = 1, _paddingX = 0, _paddingY = 0;
    int _batchNorm = 0, _useBias = 1;
    float _bnEps = 0.00001f;
    int _nWeights = 0, _nBiases = 0, _nScales = 0, _nRollMean = 0, _nRollVariance = 0;
    std::vector<float> _weights, _biases, _scales, _rollMean, _rollVariance;
};

// src/layers/MsnhBatchNormLayer.cpp:5-52, 453-480
class MsnhNet_API BatchNormLayer : public BaseLayer
{
public:
    BatchNormLayer(const int &batch, const int &width, const int &height, const int &channel, const ActivationType &activation,
                   const float &eps, const std::vector<float> &actParams);
    void loadAllWeigths(std::vector<float> &weights) override;
    void weightLayout(std::vector<long long> &parts) const override;
    int lower(Plan &plan, int in, int layerIndex) override;
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;

private:
    float _eps = 0.00001f;
    std::vector<float> _scales, _biases, _rollMean, _rollVariance;
};

// src/layers/MsnhMaxPoolLayer.cpp:5-170
class MsnhNet_API MaxPoolLayer : public BaseLayer
{
public:
    MaxPoolLayer(const int &batch, const int &height, const int &width, const int &channel, const int &kSizeX, const int &kSizeY,
                 const int &strideX, const int &strideY, const int &paddingX, const int &paddingY, const int &maxPoolDepth,
                 const int &outChannelsMp, const int &ceilMode, const int &antialiasing);
    int lower(Plan &plan, int in, int layerIndex) override;
    int getKSizeX() const { return _kSizeX; }
    int getStride() const { return _strideX; }
    int getPaddingX() const { return _paddingX; }

private:
    int _kSizeX, _kSizeY, _strideX, _strideY, _paddingX, _paddingY, _ceilMode;
};

// src/layers/MsnhLocalAvgPoolLayer.cpp:5-150
class MsnhNet_API LocalAvgPoolLayer : public BaseLayer
{
public:
    LocalAvgPoolLayer(const int &batch, const int &height, const int &width, const int &channel, const int &kSizeX, const int &kSizeY,
                      const int &strideX, const int &strideY, const int &paddingX, const int &paddingY, const int &ceilMode,
                      const int &antialiasing);
    int lower(Plan &plan, int in, int layerIndex) override;

private:
    int _kSizeX, _kSizeY, _strideX, _strideY, _paddingX, _paddingY, _ceilMode;
};

// src/layers/MsnhConnectedLayer.cpp:5-106, 495-540
class MsnhNet_API ConnectedLayer : public BaseLayer
{
public:
    ConnectedLayer(const int &batch, const int &steps, const int &inputNum, const int &outputNum, const ActivationType &activation,
                   const std::vector<float> &actParams, const int &batchNorm, const float &bnEps, const int &useBias);
    void loadAllWeigths(std::vector<float> &weights) override;
    void weightLayout(std::vector<long long> &parts) const override;
    int lower(Plan &plan, int in, int layerIndex) override;
    const std::vector<float> &kernelWeights() const override { return _weights; }
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;

private:
    int _batchNorm = 0, _useBias = 1;
    int _nWeights = 0, _nBiases = 0;
    std::vector<float> _weights, _biases;
};

// src/layers/MsnhUpSampleLayer.cpp:5-66
class MsnhNet_API UpSampleLayer : public BaseLayer
{
public:
    UpSampleLayer(const int &batch, const int &width, const int &height, const int &channel, const int &strideX, const int &strideY,
                  const float &scaleX, const float &scaleY, UpSampleParams::UpsampleType upsampleType, const int &alignCorners);
    int lower(Plan &plan, int in, int layerIndex) override;

private:
    int _strideX, _strideY;
    float _scaleX, _scaleY;
    UpSampleParams::UpsampleType _upsampleType;
    int _alignCorners;
};

// Transposed convolution (src/layers/MsnhDeConvolutionalLayer.cpp:4-70 ctor, :140-200 forward), groups == 1, square geometry.
// Lowered to a 1x1 convolution with kSize^2 * filters output channels (the reference's transposed GEMM) and a gather of the
// taps (its col2im) that also adds the bias and applies the activation.
class MsnhNet_API DeConvolutionalLayer : public BaseLayer
{
public:
    DeConvolutionalLayer(const int &batch, const int &height, const int &width, const int &channel, const int &num, const int &kSizeX,
                         const int &kSizeY, const int &strideX, const int &strideY, const int &paddingX, const int &paddingY, const int &groups,
                         const ActivationType &activation, const std::vector<float> &actParams, const int &useBias);
    ~DeConvolutionalLayer() override;
    int deConvOutHeight() const { return (_height - 1) * _strideY - 2 * _paddingY + _kSizeY; }
    int deConvOutWidth() const { return (_width - 1) * _strideX - 2 * _paddingX + _kSizeX; }
    void loadAllWeigths(std::vector<float> &weights) override;
    void weightLayout(std::vector<long long> &parts) const override;
    int lower(Plan &plan, int in, int layerIndex) override;
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;      // the bias, for the gather launch

private:
    int _kSizeX, _kSizeY, _strideX, _strideY, _paddingX, _paddingY, _useBias;
    int _nWeights = 0, _nBiases = 0;
    std::vector<float> _biases;
    BaseLayer *_gemm = nullptr;            // owner of the rearranged [k*k*filters][channel] weights of the 1x1 convolution
};

// src/layers/MsnhGlobalAvgPoolLayer.cpp:5-30, 152-168: mean of every channel plane
class MsnhNet_API GlobalAvgPoolLayer : public BaseLayer
{
public:
    GlobalAvgPoolLayer(const int &batch, const int &height, const int &width, const int &channel);
    int lower(Plan &plan, int in, int layerIndex) override;
};

// src/layers/MsnhSoftMaxLayer.cpp:5-30, 60-93 (groups == 1: one softmax over all values of an image)
class MsnhNet_API SoftMaxLayer : public BaseLayer
{
public:
    SoftMaxLayer(const int &batch, const int &inputNum, const int &groups, const float &temperature);
    int lower(Plan &plan, int in, int layerIndex) override;

private:
    int _groups;
    float _temperature;
};

// src/layers/MsnhActivationLayer.cpp:5-40 (stand-alone activation; PReLU, which owns weights, is not implemented)
class MsnhNet_API ActivationLayer : public BaseLayer
{
public:
    ActivationLayer(const int &batch, const int &width, const int &height, const int &channel, const int &inputNum,
                    const ActivationType &activation, const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;
};

// src/layers/MsnhPaddingLayer.cpp:5-45
class MsnhNet_API PaddingLayer : public BaseLayer
{
public:
    PaddingLayer(const int &batch, const int &height, const int &width, const int &channel, const int &top, const int &down,
                 const int &left, const int &right, const float &paddingVal);
    int lower(Plan &plan, int in, int layerIndex) override;

private:
    int _top, _down, _left, _right;
    float _paddingVal;
};

// src/layers/MsnhSliceLayer.cpp:5-70
class MsnhNet_API SliceLayer : public BaseLayer
{
public:
    SliceLayer(const int &batch, const int &height, const int &width, const int &channel, const int &start0, const int &step0,
               const int &start1, const int &step1, const int &start2, const int &step2);
    int lower(Plan &plan, int in, int layerIndex) override;

private:
    int _start0, _step0, _start1, _step1, _start2, _step2;
};

// src/layers/MsnhVariableOpLayer.cpp:5-60.  Implemented: add / sub / subInv of two tensors and the constant forms
// addConst / subConst / subConstInv / mulConst / divConst.
class MsnhNet_API VariableOpLayer : public BaseLayer
{
public:
    VariableOpLayer(const int &batch, const int &width, const int &height, const int &channel, std::vector<int> &inputLayerIndexes,
                    const VariableOpParams::VarOpType &varOpType, const float &constVal);
    int lower(Plan &plan, int in, int layerIndex) override;
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;
    const std::vector<int> &inputLayerIndexes() const { return _inputLayerIndexes; }

private:
    std::vector<int> _inputLayerIndexes;
    VariableOpParams::VarOpType _varOpType;
    float _constVal;
};

// src/layers/MsnhEmptyLayer.cpp (identity)
class MsnhNet_API EmptyLayer : public BaseLayer
{
public:
    EmptyLayer(const int &batch, const int &width, const int &height, const int &channel);
    int lower(Plan &plan, int in, int layerIndex) override;
};

// src/layers/MsnhRouteLayer.cpp:5-55; sizes are computed by NetBuilder (src/net/MsnhNetBuilder.cpp:205-334)
class MsnhNet_API RouteLayer : public BaseLayer
{
public:
    RouteLayer(const int &batch, std::vector<int> &inputLayerIndexes, std::vector<int> &inputLayerOutputs, const int &groups,
               const int &groupIndex, const int &addModel, const ActivationType &activation, const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
    void foldedAffine(std::vector<float> &scale, std::vector<float> &shift) const override;
    const std::vector<int> &inputLayerIndexes() const { return _inputLayerIndexes; }
    std::vector<int> inputChannels;         // channels of each routed layer, set by NetBuilder

private:
    std::vector<int> _inputLayerIndexes, _inputLayerOutputs;
    int _groups, _groupIndex, _addModel;
};

// Shared by the four block layers: builds the sub-layers of one branch exactly the way the reference's block
// constructors do (same accepted node types, same exceptions), e.g. src/layers/MsnhResBlockLayer.cpp:23-150.
class MsnhNet_API BlockLayer : public BaseLayer
{
public:
    ~BlockLayer() override;
    void loadAllWeigths(std::vector<float> &weights) override;
    void weightLayout(std::vector<long long> &parts) const override;

protected:
    std::vector<BaseLayer *> buildChain(NetBuildParams &params, std::vector<BaseParams *> &nodes, const char *blockName, bool allowEmpty);
    int lowerChain(Plan &plan, const std::vector<BaseLayer *> &chain, int in, int layerIndex);
    std::vector<std::vector<BaseLayer *>> _chains;      // weight order = chain order
};

// out = act(x + F(x))   src/layers/MsnhResBlockLayer.cpp:4-150, 215-302
class MsnhNet_API ResBlockLayer : public BlockLayer
{
public:
    ResBlockLayer(const int &batch, NetBuildParams &params, std::vector<BaseParams *> &baseParams, ActivationType &activation,
                  const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
    std::vector<BaseLayer *> &baseLayers() { return _chains[0]; }
};

// out = act(base(x) + branch(x))   src/layers/MsnhRes2BlockLayer.cpp:4-260, 342-447
class MsnhNet_API Res2BlockLayer : public BlockLayer
{
public:
    Res2BlockLayer(const int &batch, NetBuildParams &params, std::vector<BaseParams *> &baseParams, std::vector<BaseParams *> &branchParams,
                   ActivationType &activation, const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
};

// out = act(sum of branches)   src/layers/MsnhAddBlockLayer.cpp:4-250, 255-357
class MsnhNet_API AddBlockLayer : public BlockLayer
{
public:
    AddBlockLayer(const int &batch, NetBuildParams &params, std::vector<std::vector<BaseParams *>> &branchParams, ActivationType &activation,
                  const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
};

// out = act(channel concat of branches)   src/layers/MsnhConcatBlockLayer.cpp:4-250, 255-355
class MsnhNet_API ConcatBlockLayer : public BlockLayer
{
public:
    ConcatBlockLayer(const int &batch, NetBuildParams &params, std::vector<std::vector<BaseParams *>> &branchParams, ActivationType &activation,
                     const std::vector<float> &actParams);
    int lower(Plan &plan, int in, int layerIndex) override;
};

// src/layers/MsnhYoloLayer.cpp:5-58
class MsnhNet_API YoloLayer : public BaseLayer
{
public:
    YoloLayer(const int &batch, const int &width, const int &height, const int &num, const int &orgWidth, const int &orgHeight,
              const int &classNum, const std::vector<float> &anchors, const YoloType &yoloType);
    int lower(Plan &plan, int in, int layerIndex) override;
    int getClassNum() const { return _classNum; }
    float getRatios() const { return _ratios; }
    YoloType getYoloType() const { return _yoloType; }
    std::vector<float> anchors;
    int cellBase = 0;          // set by the YoloOutLayer that consumes this head
    float confThresh = 2.f;    // likewise; 2 = "no candidate list" until a yoloout claims the head
    size_t decodeOp = 0;

private:
    int _orgHeight, _orgWidth, _classNum;
    float _ratios;
    YoloType _yoloType;
};

// src/layers/MsnhYoloOutLayer.cpp:4-60 (ctor), :79-203 (candidate scan + sort), :381-461 (nms)
class MsnhNet_API YoloOutLayer : public BaseLayer
{
public:
    YoloOutLayer(const int &batch, const int &orgWidth, const int &orgHeight, std::vector<int> &yoloIndexes, std::vector<YoloInfo> &yoloLayersInfo,
                 const float &confThresh, const float &nmsThresh, const int &useSotfNms, const YoloType &yoloType);
    ~YoloOutLayer() override;
    int lower(Plan &plan, int in, int layerIndex) override;
    void forwardGPU(NetworkState &netState) override;      // device candidate compaction + host sort / NMS
    // The three stages of forwardGPU, separately, so that a caller can overlap the host stage of one batch with
    // the device work of the next (two copy-back slots):
    void enqueueGather(msnh_stream_t s);                   // device: compact the candidate rows
    void enqueueCopyBack(msnh_stream_t s, int slot);       // device -> pinned host, asynchronous
    void finish(int slot);                                 // host: wait, sort, NMS -> finalOut

    static std::vector<YoloBox> nms(const std::vector<YoloBox> &bboxes, const float &nmsThresh, const bool &useSoftNms, const float &sigma = 0.3f);
    // hard NMS with the same result as nms(), restructured for speed (see the definition)
    static std::vector<YoloBox> nmsSorted(const std::vector<YoloBox> &bboxes, float nmsThresh);
    // boxes from network-input pixels back to the original image (reference: MsnhYoloOutLayer.cpp:321-379)
    static YoloBox bboxResize2Org(YoloBox &box, const Point2I &currentShape, const Point2I &orgShape);
    static YoloBox bboxResize2OrgNoPad(YoloBox &box, const Point2I &currentShape, const Point2I &orgShape);
    float getConfThresh() const { return _confThresh; }
    float getNmsThresh() const { return _nmsThresh; }
    int   getUseSoftNms() const { return _useSoftNms; }
    YoloType getYoloType() const { return _yoloType; }
    const std::vector<int> &yoloIndexes() const { return _yoloIndexes; }

    std::vector<bool> batchHasBox;
    std::vector<std::vector<YoloBox>> finalOut;
    static bool keepClassScores;           // also fill YoloBox::classesVal (costs an extra device->host copy)
    bool lastOnDevice = false;             // where the NMS of the result fetched last ran
    bool copyOnForwardStream = false;      // copy-back (and device NMS) on the forward's stream instead of a stream of their own (NetGroup)
    // hard NMS on the device (only the kept boxes are copied back): 0 = never (sort + NMS on the host), 2 = always,
    // 1 (default) = chosen per batch from the previous result: up to kDeviceNmsFew candidates per image on the device; up to
    // kDeviceNmsCandidates (the largest class the device kernels take) on the device as well, except while forwards are pipelined and
    // the host stage keeps up with them -- the host then does it for free beside the next forward; more than that on the host.
    // "Keeps up" is measured: when the host stage stops waiting for the device, kTrialBatches batches run on the device and the
    // placement with the shorter time between results stays.
    static int deviceNms;
    static const int kDeviceNmsFew = 2048;
    static const int kDeviceNmsCandidates = 6144;
    static const int kTrialBatches = 16;

    // host post-processing of the compacted candidate rows of one image (8 floats per row, see msnh_hip_yolo_gather)
    std::vector<YoloBox> boxesFromRows(const float *rows, int count, const float *decodedOfImage) const;
    // the same as a function of the rows alone: candidates back in scan order (by cell number), then sorted by objectness * class score,
    // descending, ties in scan order (src/layers/MsnhYoloOutLayer.cpp:120-194); decodedOfImage (may be NULL) supplies classesVal
    static std::vector<YoloBox> sortedCandidates(const float *rows, int count, const float *decodedOfImage, int channel);
    // the candidate rows of image `image` in the result fetched last, as the device wrote them (8 floats each: x y w h objectness, best
    // class score, best class, cell number in scan order; any order) -- what the reference's scan keeps before sorting
    // (src/layers/MsnhYoloOutLayer.cpp:120-170).  Only after a result whose sort + NMS ran on the host.
    std::vector<float> lastCandidateRows(int image) const;
    // one line for NetBuilder::getTimeDetail: where the sort + NMS of the last result ran and what the automatic placement has measured
    std::string placementDetail() const;
    static std::vector<std::vector<int>> groupByClass(const std::vector<YoloBox> &bboxes);
    static void nmsClass(const std::vector<YoloBox> &bboxes, std::vector<int> &members, float nmsThresh);

private:
    float _confThresh, _nmsThresh;
    int _useSoftNms, _orgHeight, _orgWidth;
    YoloType _yoloType;
    std::vector<int> _yoloIndexes;
    std::vector<YoloInfo> _yoloLayersInfo;
    int _yoloAllInputNum = 0, _pixels = 0;
    // devCnt / devRows: device-side snapshot of one forward's candidates, so the copy to the host can run on its own
    // stream while the next forward already overwrites the plan's buffers
    struct Slot
    {
        PinnedBuffer cnt, rows, decoded, kept, keptCnt;
        DeviceBuffer devCnt, devRows, devKept, devKeptCnt, devNmsWs;
        msnh_event_t event = nullptr, ready = nullptr;
        bool pending = false, onDevice = false;
        bool trial = false;                // part of a device trial of the automatic placement
        size_t rowsCopied = 0;             // row slots per image that the asynchronous copy brings to the host
        size_t quick = 0;                  // device NMS: records that the asynchronous copy brings to the host
    };
    std::vector<YoloBox> boxesFromKept(std::vector<const float *> &records) const;
    msnh_stream_t _copyStream = nullptr, _fetchStream = nullptr;
    int _lastMaxCandidates = 0;            // largest per-image candidate count of the previous result
    int _lastSlot = -1;                    // slot of the result fetched last
    size_t _lastKept = 0;                  // records the device NMS kept for the previous batch
    int _hostBoundRuns = 0;                // batches in a row for which the host path did not have to wait for the device
    bool _hostBound = false;               // a device trial gave results faster than the host stage: stay on the device
    int _trialLeft = 0, _trialSeen = 0, _trialSamples = 0;   // device trial: batches to enqueue / finished / intervals measured
    double _trialSum = 0.0, _hostInterval = 0.0;             // ms between results: sum over the trial, moving mean of the host mode
    std::chrono::steady_clock::time_point _lastFinish;
    bool _haveLastFinish = false, _lastFinishHost = false;
    void noteResult(const Slot &sl, bool pipelined);
    void prepareSlot(Slot &sl, bool deviceNmsBuffers);
    Slot _slots[2];
};
}
