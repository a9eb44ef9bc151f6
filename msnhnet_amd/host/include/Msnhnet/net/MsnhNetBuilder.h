// NetBuilder: build a network from a `.msnhnet` file, load `.msnhbin` weights, run it.
// Public interface = the reference's (include/Msnhnet/net/MsnhNetBuilder.h:48-117) with the GPU entry points
// unconditional.  Extensions, all optional: batches larger than one (the reference rejects them),
// setKeepClassScores, the last-run accessors used by tests and the benchmark.
#pragma once
#include <string>
#include <vector>
#include "Msnhnet/io/MsnhParser.h"
#include "Msnhnet/layers/MsnhLayers.h"
#include "Msnhnet/net/MsnhNetwork.h"

namespace Msnhnet
{
class MsnhNet_API NetBuilder
{
public:
    NetBuilder();
    ~NetBuilder();

    static void setPreviewMode(const bool &mode);
    static void setMemAlign(const bool &memAlign);
    static void setOnlyGpu(const bool &onlyGpu);
    static void setOnlyCpu(const bool &onlyCpu);
    static void setUseFp16(const bool &useFp16);
    static void setForceUseCuda(const bool &onlyUseCuda);
    static void setKeepClassScores(const bool &keep);
    // Per-layer search for the fastest convolution tile configuration at load time (default on).
    static void setAutoTune(const bool &on);
    // keep the per-layer tile / algorithm choices next to the weights file ("<path>.msnhbin.tune"): the next load of the same
    // graph on the same device skips the search.  Off by default (the library then writes no files).
    // hard NMS of detection networks: 0 = candidates are copied back and sorted / suppressed on the host, 2 = on the device (only
    // kept boxes are copied back), 1 (default) = on the device while the previous result had at most 2048 candidates per image
    static void setDeviceNms(const int &mode);
    static void setTuneCache(const bool &on);
    static bool tuneCache;
    // keep the packed device-side kernels and the float16 calibration in "<weights>.f16.pack" / ".f32.pack" beside the weights file: the next
    // load of the same weights into the same graph uploads them as they are (no calibration pass, no re-packing)
    static void setWeightCache(const bool &on);
    static bool weightCache;
    static void setUseWinograd(const bool &on);   // float16 plans: 3x3 stride-1 convolutions through Winograd F(2x2,3x3)
    static bool useWinograd;
    static bool autoTune;

    void buildNetFromMsnhNet(const std::string &path);
    void loadWeightsFromMsnhBin(const std::string &path);
    void loadWeightsFromVector(const std::vector<float> &weights);     // same slicing, no file

    // The reference's CPU entry points: this build has no CPU path, they throw "Gpu mode , can not run with cpu".
    std::vector<float> runClassify(std::vector<float> img);
    std::vector<std::vector<YoloBox>> runYolo(std::vector<float> img);
    // img holds batch*C*H*W floats, batch-major NCHW (one image when the graph's batch is 1, as in the reference).
    std::vector<float> runClassifyGPU(std::vector<float> img);
    std::vector<std::vector<YoloBox>> runYoloGPU(std::vector<float> img);
    // the same two calls on a caller's buffer of `count` floats (what the C ABI holds: no vector is built from it)
    std::vector<float> runClassifyGPU(const float *img, size_t count);
    std::vector<std::vector<YoloBox>> runYoloGPU(const float *img, size_t count);

    // Steady-state serving path: the input already lives on the device (NCHW float32, batch*C*H*W floats).
    // Enqueues one forward on the builder's stream; results are fetched with fetchClassify / fetchYolo.
    // Detection networks may have two forwards in flight (enqueue, enqueue, fetch, enqueue, fetch, ...): the
    // host-side sort / NMS of one batch then overlaps the device work of the next.
    void enqueueForward(const float *deviceInput);
    void sync();
    std::vector<float> fetchClassify();
    std::vector<std::vector<YoloBox>> fetchYolo();
    float *deviceInputBuffer();               // the builder's own device input buffer (batch*C*H*W floats)
    // Letterboxes one 8-bit RGB image (HWC, host memory) on the device into slot `index` of the input batch: what
    // CVUtil::getPaddingZeroF32C3 + the float upload do in the reference (MsnhCVUtil.cpp:203-261); then
    // enqueueForward(nullptr) runs on it.
    void setInputImageU8(int index, const unsigned char *rgbHwc, int width, int height, bool halfInit = false, bool shuffleRGB = false);
    // The same with any of the reference's 8-bit pre-processing variants (msnh_preproc: CVUtil::getImgDataF32C3,
    // getGoogLenetF32C3, getTransformedF32C3, getCaffeModeF32C3 or the letterbox; MsnhCVUtil.cpp:91-375) resized to the
    // network's input size on the device.  mean / std: three floats each, only read by MSNH_PRE_TRANSFORMED.
    void setInputImage(int index, const unsigned char *rgbHwc, int width, int height, int preproc, const float *mean, const float *std, bool shuffleRGB);

    // Range check of the float16 plan for one input (batch*C*H*W floats): the activation scales are fixed at load from one
    // calibration image of values in [0,1) with a 32x margin; this runs the network once, launch by launch, on `img` and returns the
    // factor by which `img` could still grow before a float16 activation overflows (0: it already did; the results are then wrong).
    // Detectors, after a fetched result: the input of detection head `head` (heads in the order of the yoloout layer's `layers:` list)
    // as batch-major NCHW float32 -- the tensor the reference's YoloLayer::forward reads (src/layers/MsnhYoloLayer.cpp:61-142) -- and the
    // candidate rows of one image before sorting and suppression (YoloOutLayer::lastCandidateRows).  For parity checks of the
    // production path: which cells passed the objectness test, and on which logits.
    std::vector<float> yoloHeadLogits(int head);
    std::vector<float> yoloLastCandidates(int image);
    float fp16Headroom(const std::vector<float> &img);

    Point2I getInputSize();
    int getInputChannel();
    int getBatch() const;
    bool lastNmsOnDevice() const;           // detection networks: where the NMS of the result fetched last ran (see YoloOutLayer::deviceNms)
    void clearLayers();
    float getInferenceTime();
    std::string getLayerDetail();
    std::string getTimeDetail();
    float getGpuInferenceTime() const;
    Network *getNet() const;
    int getLastLayerOutWidth() const;
    int getLastLayerOutHeight() const;
    int getLastLayerOutChannel() const;
    size_t getLastLayerOutNum() const;
    void setSaveLayerOutput(bool saveLayerOutput);
    bool getSaveLayerWeights() const;
    void setSaveLayerWeights(bool saveLayerWeights);

    // When layer dumps are on, the last run's per-layer outputs are kept here (batch-major NCHW float32)
    // instead of being written to "<i>gpu.txt" files only.
    const std::vector<std::vector<float>> &layerOutputs() const { return _layerOutputs; }
    void setWriteDumpFiles(bool on) { _writeDumpFiles = on; }
    std::string getPlanDetail() const;
    std::string getLoadDetail() const;      // wall-clock of the phases of the last load, and what happened to the pack file
    double getConvFlops() const;              // 2*MACs of all conv/connected launches of one forward (whole batch)
    // Times `reps` eager passes over the live ops of one kind (PlanOp::Kind, or -1 for all) with device events on
    // the builder's stream; returns the total milliseconds and the number of launches timed.  The ops run on
    // whatever the buffers currently hold, so this is a timing tool, not a forward.  kind 1000 + a: the convolution launches of
    // algorithm a (MSNH_CONV_*).  bytes (optional): what those launches must move at least (input + output + residual + weights).
    float profileOps(int kind, int reps, int *launches, double *flops, double *bytes = nullptr);
    // One line per live op: layer, kind, shapes, algorithm, microseconds per launch (mean of `reps`), TFLOP/s, GB/s.
    // every live launch of the plan timed on its own (reps back-to-back repetitions); values (optional) receives 8 numbers per launch:
    // kind, algorithm, layer index, tile, algorithmic FLOPs, least bytes (input + output + fused residual + weights), microseconds, ksize * 100 + stride
    std::string profileEachOp(int reps, std::vector<double> *values = nullptr);

private:
    void finalizePlan();
    std::string _weightsPath;               // set while loadWeightsFromMsnhBin runs: where the tune cache goes
    uint64_t _graphTextHash = 0, _weightsHash = 0;
    float _readMs = 0.f;
    std::string _loadDetail;
    std::unique_ptr<Plan> lowerNetwork(int dtype);
    void uploadInput(const float *img, size_t count);
    void runLayersEager();
    void checkInput(size_t given) const;

    Parser       *_parser;
    Network      *_net;
    NetworkState *_netState;
    float  _gpuInferenceTime = 0.f;
    int    _lastLayerOutWidth = 0, _lastLayerOutHeight = 0, _lastLayerOutChannel = 0;
    size_t _lastLayerOutNum = 0;
    bool   _saveLayerOutput = false, _saveLayerWeights = false, _writeDumpFiles = false;
    bool   _planReady = false;
    std::vector<std::vector<float>> _layerOutputs;
    DeviceBuffer _inputDev, _imageDev;
    PinnedBuffer _imagePinned;
    PinnedBuffer _inputPinned, _outputPinned;
    msnh_stream_t _stream = nullptr;
    msnh_graph_t  _graph = nullptr;
    const float  *_graphInput = nullptr;
    int _nextSlot = 0, _inFlight = 0;          // copy-back slots of the detection post-processing
};
}
