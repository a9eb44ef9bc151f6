// NetBuilder: graph construction, weight loading, planning and the run entry points.
// Control flow and error texts follow src/net/MsnhNetBuilder.cpp of the reference (build :68-622, load :624-663,
// run :820-1007); what happens underneath -- one planned device arena, fused launches, a captured graph --
// is new.
#include <cstdlib>
#include "Msnhnet/net/MsnhNetBuilder.h"
#include "Msnhnet/utils/MsnhTaskPool.h"
#include <chrono>
#include <cmath>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>

namespace Msnhnet
{
void Network::forward(NetworkState &) { MSNH_THROW("Gpu mode , can not run with cpu"); }

void Network::forwardGPU(NetworkState &netState)
{
    for (BaseLayer *l : layers) l->forwardGPU(netState);
}

NetBuilder::NetBuilder()
{
    _parser = new Parser();
    _net = new Network();
    _netState = new NetworkState();
    _netState->net = _net;
}

NetBuilder::~NetBuilder()
{
    clearLayers();
    if (_stream) msnh_hip_stream_destroy(_stream);
    delete _netState;
    delete _net;
    delete _parser;
}

void NetBuilder::setPreviewMode(const bool &mode) { BaseLayer::setPreviewMode(mode); }
void NetBuilder::setMemAlign(const bool &memAlign) { BaseLayer::setMemAlign(memAlign); }
void NetBuilder::setOnlyGpu(const bool &onlyGpu) { BaseLayer::setOnlyGpu(onlyGpu); }
void NetBuilder::setUseFp16(const bool &useFp16) { BaseLayer::setUseFp16(useFp16); }
void NetBuilder::setForceUseCuda(const bool &v) { BaseLayer::setForceUseCuda(v); }
void NetBuilder::setKeepClassScores(const bool &keep) { YoloOutLayer::keepClassScores = keep; }
void NetBuilder::setDeviceNms(const int &mode)
{
    if (mode < 0 || mode > 2) throw Exception(1, "setDeviceNms: mode must be 0 (host), 1 (by candidate count) or 2 (device)", __FILE__, __LINE__, __FUNCTION__);
    YoloOutLayer::deviceNms = mode;
}
bool NetBuilder::autoTune = true;
void NetBuilder::setAutoTune(const bool &on) { autoTune = on; }
bool NetBuilder::tuneCache = false;
void NetBuilder::setTuneCache(const bool &on) { tuneCache = on; }
bool NetBuilder::weightCache = false;
void NetBuilder::setWeightCache(const bool &on) { weightCache = on; }
bool NetBuilder::useWinograd = false;
void NetBuilder::setUseWinograd(const bool &on) { useWinograd = on; }

void NetBuilder::setOnlyCpu(const bool &onlyCpu)
{
    if (onlyCpu) MSNH_THROW("cpu only mode is not available: this build has no CPU compute path");
    BaseLayer::setOnlyCpu(false);
}

void NetBuilder::clearLayers()
{
    if (_graph) { msnh_hip_graph_destroy(_graph); _graph = nullptr; }
    _net->plan.reset();
    for (BaseLayer *l : _net->layers) delete l;
    _net->layers.clear();
    _planReady = false;
    _layerOutputs.clear();
    _nextSlot = 0;
    _inFlight = 0;
}

// ---- build -----------------------------------------------------------------------------------------------------------
void NetBuilder::buildNetFromMsnhNet(const std::string &path)
{
    _parser->readCfg(path);
    {
        // every parameter of the graph (activation slopes, batch-norm eps, anchors, thresholds, ...) takes part in what a packed-constants
        // file must match: the file keeps a float16 calibration that depends on them
        std::ifstream f(path, std::ios::binary);
        const std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        _graphTextHash = PackFile::hash(text.data(), text.size());
    }
    clearLayers();
    if (BaseLayer::onlyUseGpu && BaseLayer::onlyUseCpu) MSNH_THROW("Gpu only mode and cpu only mode can not use at the same time!");

    NetBuildParams params;
    for (size_t i = 0; i < _parser->params.size(); ++i)
    {
        BaseParams *bp = _parser->params[i];
        BaseLayer *layer = nullptr;
        if (i == 0)
        {
            if (bp->type != LayerType::CONFIG) MSNH_THROW("The first params must be config");
            NetConfigParams *cfg = static_cast<NetConfigParams *>(bp);
            if (cfg->height <= 0 || cfg->width <= 0 || cfg->channels <= 0 || cfg->batch <= 0) MSNH_THROW("net config params err, params = 0 or < 0");
            _net->batch = cfg->batch; _net->channels = cfg->channels; _net->width = cfg->width; _net->height = cfg->height;
            _net->inputNum = _net->batch * _net->channels * _net->width * _net->height;
            params.height = _net->height; params.batch = _net->batch; params.width = _net->width; params.channels = _net->channels;
            params.inputNums = _net->inputNum;
            continue;
        }
        const size_t nLayers = _net->layers.size();
        switch (bp->type)
        {
        case LayerType::CONVOLUTIONAL:
        {
            if (params.height == 0 || params.width == 0 || params.channels == 0) MSNH_THROW("Layer before convolutional layer must output image");
            ConvParams *p = static_cast<ConvParams *>(bp);
            layer = new ConvolutionalLayer(params.batch, 1, params.height, params.width, params.channels, p->filters, p->groups, p->kSizeX, p->kSizeY,
                                           p->strideX, p->strideY, p->dilationX, p->dilationY, p->paddingX, p->paddingY, p->activation, p->actParams,
                                           p->batchNorm, p->bnEps, p->useBias, 0, 0, 0, 0, p->antialiasing, nullptr, 0, 0);
            break;
        }
        case LayerType::CONNECTED:
        {
            ConnectParams *p = static_cast<ConnectParams *>(bp);
            // inputs of one sample (the reference's batch-1 files make params.inputNums exactly that)
            layer = new ConnectedLayer(params.batch, 1, params.height * params.width * params.channels, p->output, p->activation, p->actParams,
                                       p->batchNorm, p->bnEps, p->useBias);
            break;
        }
        case LayerType::MAXPOOL:
        {
            MaxPoolParams *p = static_cast<MaxPoolParams *>(bp);
            layer = new MaxPoolLayer(params.batch, params.height, params.width, params.channels, p->kSizeX, p->kSizeY, p->strideX, p->strideY, p->paddingX,
                                     p->paddingY, p->maxPoolDepth, p->outChannels, p->ceilMode, 0);
            break;
        }
        case LayerType::LOCAL_AVGPOOL:
        {
            LocalAvgPoolParams *p = static_cast<LocalAvgPoolParams *>(bp);
            layer = new LocalAvgPoolLayer(params.batch, params.height, params.width, params.channels, p->kSizeX, p->kSizeY, p->strideX, p->strideY,
                                          p->paddingX, p->paddingY, p->ceilMode, 0);
            break;
        }
        case LayerType::BATCHNORM:
        {
            BatchNormParams *p = static_cast<BatchNormParams *>(bp);
            layer = new BatchNormLayer(params.batch, params.width, params.height, params.channels, p->activation, p->eps, p->actParams);
            break;
        }
        case LayerType::RES_BLOCK:
        {
            ResBlockParams *p = static_cast<ResBlockParams *>(bp);
            layer = new ResBlockLayer(params.batch, params, p->baseParams, p->activation, p->actParams);
            break;
        }
        case LayerType::RES_2_BLOCK:
        {
            Res2BlockParams *p = static_cast<Res2BlockParams *>(bp);
            layer = new Res2BlockLayer(params.batch, params, p->baseParams, p->branchParams, p->activation, p->actParams);
            break;
        }
        case LayerType::ADD_BLOCK:
        {
            AddBlockParams *p = static_cast<AddBlockParams *>(bp);
            layer = new AddBlockLayer(params.batch, params, p->branchParams, p->activation, p->actParams);
            break;
        }
        case LayerType::CONCAT_BLOCK:
        {
            ConcatBlockParams *p = static_cast<ConcatBlockParams *>(bp);
            layer = new ConcatBlockLayer(params.batch, params, p->branchParams, p->activation, p->actParams);
            break;
        }
        case LayerType::EMPTY:
            layer = new EmptyLayer(params.batch, params.width, params.height, params.channels);
            break;
        case LayerType::ROUTE:
        {
            RouteParams *p = static_cast<RouteParams *>(bp);
            if (p->layerIndexes.size() < 1) MSNH_THROW("route layer error, no route layers");
            std::vector<int> outputs, chans;
            int outC = 0, outH = 0, outW = 0;
            for (size_t k = 0; k < p->layerIndexes.size(); ++k)
            {
                const int idx = p->layerIndexes[k];
                if (idx < 0 || static_cast<size_t>(idx) >= nLayers) MSNH_THROW("route layer error, route layers index should < size of layers");
                const BaseLayer *src = _net->layers[static_cast<size_t>(idx)];
                if (k > 0 && (src->getOutHeight() != outH || src->getOutWidth() != outW))
                {
                    std::string indexes;
                    for (int v : p->layerIndexes) indexes += std::to_string(v) + ", ";
                    MSNH_THROW("[route] layers height or width not equal. layer: " + std::to_string(i - 1) + "  aux: " + indexes + "wh: " +
                               std::to_string(outW) + ":" + std::to_string(src->getOutWidth()) + " , " + std::to_string(outH) + ":" +
                               std::to_string(src->getOutHeight()) + " ");
                }
                if (p->addModel == 1 && k > 0 && src->getOutChannel() != outC)
                    MSNH_THROW("[route] layers height or width not equal. layer: " + std::to_string(i - 1) + " whc: channels " + std::to_string(outC) + ":" +
                               std::to_string(src->getOutChannel()));
                outH = src->getOutHeight(); outW = src->getOutWidth();
                if (p->addModel == 1) outC = src->getOutChannel();
                else outC += src->getOutChannel();
                outputs.push_back(src->getOutputNum());
                chans.push_back(src->getOutChannel());
            }
            RouteLayer *r = new RouteLayer(params.batch, p->layerIndexes, outputs, p->groups, p->groupsId, p->addModel, p->activation, p->actParams);
            r->inputChannels = chans;
            r->setOutChannel(outC); r->setOutWidth(outW); r->setOutHeight(outH);
            layer = r;
            break;
        }
        case LayerType::DECONVOLUTIONAL:
        {
            if (params.height == 0 || params.width == 0 || params.channels == 0) MSNH_THROW("Layer before deconvolutional layer must output image");
            DeConvParams *p = static_cast<DeConvParams *>(bp);
            layer = new DeConvolutionalLayer(params.batch, params.height, params.width, params.channels, p->filters, p->kSizeX, p->kSizeY, p->strideX,
                                             p->strideY, p->paddingX, p->paddingY, p->groups, p->activation, p->actParams, p->useBias);
            break;
        }
        case LayerType::GLOBAL_AVGPOOL:
            layer = new GlobalAvgPoolLayer(params.batch, params.height, params.width, params.channels);
            break;
        case LayerType::SOFTMAX:
        {
            SoftMaxParams *p = static_cast<SoftMaxParams *>(bp);
            layer = new SoftMaxLayer(params.batch, params.inputNums, p->groups, p->temperature);
            break;
        }
        case LayerType::ACTIVE:
        {
            ActivationParams *p = static_cast<ActivationParams *>(bp);
            layer = new ActivationLayer(params.batch, params.width, params.height, params.channels, params.inputNums, p->activation, p->actParams);
            break;
        }
        case LayerType::PADDING:
        {
            PaddingParams *p = static_cast<PaddingParams *>(bp);
            layer = new PaddingLayer(params.batch, params.height, params.width, params.channels, p->top, p->down, p->left, p->right, p->paddingVal);
            break;
        }
        case LayerType::SLICE:
        {
            SliceParams *p = static_cast<SliceParams *>(bp);
            layer = new SliceLayer(params.batch, params.height, params.width, params.channels, p->start0, p->step0, p->start1, p->step1, p->start2, p->step2);
            break;
        }
        case LayerType::VARIABLE_OP:
        {
            VariableOpParams *p = static_cast<VariableOpParams *>(bp);
            for (int idx : p->layerIndexes)
                if (idx < 0 || static_cast<size_t>(idx) >= nLayers) MSNH_THROW("varop layer error, layers index should < size of layers");
            layer = new VariableOpLayer(params.batch, params.width, params.height, params.channels, p->layerIndexes, p->varOpType, p->constVal);
            break;
        }
        case LayerType::UPSAMPLE:
        {
            UpSampleParams *p = static_cast<UpSampleParams *>(bp);
            layer = new UpSampleLayer(params.batch, params.width, params.height, params.channels, p->strideX, p->strideY, p->scaleX, p->scaleY,
                                      p->upsampleType, p->alignCorners);
            break;
        }
        case LayerType::YOLO:
        {
            YoloParams *p = static_cast<YoloParams *>(bp);
            layer = new YoloLayer(params.batch, params.width, params.height, params.channels, p->orgWidth, p->orgHeight, p->classNum, p->anchors, p->yoloType);
            break;
        }
        case LayerType::YOLO_OUT:
        {
            YoloOutParams *p = static_cast<YoloOutParams *>(bp);
            if (p->layerIndexes.size() < 1) MSNH_THROW("yoloOut layer error, no yolo layers");
            std::vector<YoloInfo> infos;
            for (int idx : p->layerIndexes)
            {
                if (idx < 0 || static_cast<size_t>(idx) >= nLayers) MSNH_THROW("yoloout layer error, yolo layers index should < size of layers");
                const BaseLayer *src = _net->layers[static_cast<size_t>(idx)];
                if (src->type() != LayerType::YOLO) MSNH_THROW("yoloout layer error, not a yolo layer");
                infos.push_back(YoloInfo(src->getOutHeight(), src->getOutWidth(), src->getOutChannel()));
            }
            layer = new YoloOutLayer(params.batch, p->orgWidth, p->orgHeight, p->layerIndexes, infos, p->confThresh, p->nmsThresh, p->useSoftNms, p->yoloType);
            break;
        }
        default:
            MSNH_THROW("layer type " + std::to_string(static_cast<int>(bp->type)) + " is outside the convolutional path this build implements");
        }
        params.height = layer->getOutHeight();
        params.width = layer->getOutWidth();
        params.channels = layer->getOutChannel();
        params.inputNums = layer->getOutputNum();
        layer->setLayerIndex(static_cast<int>(i) - 1);
        _net->layers.push_back(layer);
    }
    if (_net->layers.empty()) MSNH_THROW("the network has no layers");
    BaseLayer *last = _net->layers.back();
    _lastLayerOutHeight = last->getOutHeight(); _lastLayerOutWidth = last->getOutWidth(); _lastLayerOutChannel = last->getOutChannel();
    _lastLayerOutNum = static_cast<size_t>(last->getOutputNum());
}

// ---- weights ---------------------------------------------------------------------------------------------------------
void NetBuilder::loadWeightsFromMsnhBin(const std::string &path)
{
    if (BaseLayer::isPreviewMode) MSNH_THROW("Can not load weights in preview mode !");
    const auto t0 = std::chrono::steady_clock::now();
    _parser->readMsnhBin(path);
    _weightsPath = path;
    _weightsHash = weightCache ? PackFile::hash(_parser->msnhF32Weights.data(), _parser->msnhF32Weights.size() * sizeof(float)) : 0;
    _readMs = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
    loadWeightsFromVector(_parser->msnhF32Weights);
    _weightsPath.clear();
    std::vector<float>().swap(_parser->msnhF32Weights);
}

void NetBuilder::loadWeightsFromVector(const std::vector<float> &all)
{
    if (BaseLayer::isPreviewMode) MSNH_THROW("Can not load weights in preview mode !");
    size_t ptr = 0;
    for (BaseLayer *l : _net->layers)
    {
        const LayerType t = l->type();
        const bool has = t == CONVOLUTIONAL || t == DECONVOLUTIONAL || t == CONNECTED || t == BATCHNORM || t == RES_BLOCK || t == RES_2_BLOCK || t == ADD_BLOCK || t == CONCAT_BLOCK;
        if (!has) continue;
        const size_t n = l->getNumWeights();
        if (ptr + n > all.size())
            MSNH_THROW("Load weights err, need > given. Needed :" + std::to_string(ptr + n) + " given :" + std::to_string(all.size()));
        std::vector<float> part(all.begin() + static_cast<long long>(ptr), all.begin() + static_cast<long long>(ptr + n));
        l->loadAllWeigths(part);
        ptr += n;
    }
    if (ptr != all.size()) MSNH_THROW("Load weights err, need != given. Needed :" + std::to_string(ptr) + " given :" + std::to_string(all.size()));
    if (_weightsPath.empty()) _readMs = 0.f;
    finalizePlan();
}

// ---- planning --------------------------------------------------------------------------------------------------------
std::unique_ptr<Plan> NetBuilder::lowerNetwork(int dtype)
{
    std::unique_ptr<Plan> plan(new Plan(dtype));
    plan->inputTensor = plan->addTensor(_net->batch, _net->height, _net->width, _net->channels, MSNH_F32, "input", PlanTensor::NCHW_INPUT);
    plan->tensors[static_cast<size_t>(plan->inputTensor)].external = true;
    plan->tensors[static_cast<size_t>(plan->inputTensor)].extPtr = _inputDev.ptr();
    int cur = plan->inputTensor;
    for (size_t i = 0; i < _net->layers.size(); ++i)
    {
        BaseLayer *l = _net->layers[i];
        const size_t before = plan->ops.size();
        if (l->type() != LayerType::CONVOLUTIONAL && l->type() != LayerType::ROUTE && l->type() != LayerType::YOLO_OUT &&
            plan->tensors[static_cast<size_t>(cur)].layout == PlanTensor::NCHW_INPUT)
        {
            // any first layer other than a conv reads NHWC: convert the input once
            const int cast = plan->addTensor(_net->batch, _net->height, _net->width, _net->channels, dtype, "input_nhwc");
            plan->addOp(PlanOp::INPUT_CAST, cur, -1, cast, static_cast<int>(i), "input_cast");
            cur = cast;
        }
        cur = l->lower(*plan, cur, static_cast<int>(i));
        plan->layerOut.push_back(cur);
        (void)before;
        if (_saveLayerOutput) plan->tensors[static_cast<size_t>(cur)].pinned = true;
    }
    // whatever the caller can still ask for after the forward must survive it
    plan->tensors[static_cast<size_t>(plan->layerOut.back())].persistent = true;
    for (size_t i = 0; i < _net->layers.size(); ++i)
        if (_saveLayerOutput) plan->tensors[static_cast<size_t>(plan->layerOut[i])].persistent = true;
    return plan;
}

static void setupYoloBuffers(Plan &plan, int batch)
{
    if (plan.yoloCells <= 0)
    {
        // yolo layers without a yoloout still need somewhere to decode into
        int cells = 0;
        for (PlanOp &op : plan.ops)
            if (op.kind == PlanOp::YOLO_DECODE)
            {
                const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
                op.cellBase = cells;
                cells += 3 * in.h * in.w;
                plan.yoloClasses = op.classes;
            }
        plan.yoloCells = cells;
    }
    if (plan.yoloCells <= 0) return;
    const size_t per = static_cast<size_t>(5 + plan.yoloClasses);
    const size_t cells = static_cast<size_t>(plan.yoloCells);
    plan.yoloDecoded.alloc(sizeof(float) * cells * per * static_cast<size_t>(batch));
    plan.yoloCandIdx.alloc(sizeof(int) * cells * static_cast<size_t>(batch));
    plan.yoloCandCnt.alloc(sizeof(int) * static_cast<size_t>(std::max(batch, 64)));
    plan.yoloRows.alloc(sizeof(float) * 8 * cells * static_cast<size_t>(batch));
    plan.findYoloHeads();
}

void NetBuilder::finalizePlan()
{
    Device::ensureInit();
    if (_stream == nullptr) MSNH_DEV(msnh_hip_stream_create(&_stream));
    _netState->stream = _stream;
    const size_t inBytes = sizeof(float) * static_cast<size_t>(_net->inputNum);
    if (_inputDev.bytes() < inBytes) _inputDev.alloc(inBytes);
    _inputPinned.reserve(inBytes);
    _netState->gpuInput = _inputDev.as<float>();
    if (_graph) { msnh_hip_graph_destroy(_graph); _graph = nullptr; }
    _nextSlot = 0;
    _inFlight = 0;

    using Clock = std::chrono::steady_clock;
    const auto msSince = [](Clock::time_point t) { return std::chrono::duration<float, std::milli>(Clock::now() - t).count(); };
    Clock::time_point t0 = Clock::now();
    const int dtype = BaseLayer::useFp16 ? MSNH_F16 : MSNH_F32;
    std::unique_ptr<Plan> plan = lowerNetwork(dtype);
    plan->fuseStemDown = std::getenv("MSNH_NO_STEM_DOWN") == nullptr;
    plan->fuseMbconv = std::getenv("MSNH_NO_MBCONV") == nullptr;
    plan->fuseStemTail = std::getenv("MSNH_NO_STEM_TAIL") == nullptr;
    plan->fuseUpsample = std::getenv("MSNH_NO_CONV_UPSAMPLE") == nullptr;
    // (measured level with two launches inside a forward, so not the default: MSNH_CONV_TAIL=1 lets the load-time search decide per pair,
    // MSNH_FORCE_CONV_TAIL=1 takes every pair the library accepts)
    plan->forceTail = std::getenv("MSNH_FORCE_CONV_TAIL") != nullptr;
    plan->fuseTail = plan->forceTail || std::getenv("MSNH_CONV_TAIL") != nullptr;
    plan->fuse();
    plan->chainMaxPools();
    plan->aliasConcats();
    const float lowerMs = msSince(t0);

    // The packed kernels and the calibration of an earlier load of these weights into this graph, if asked for and still valid
    const bool winograd = useWinograd && dtype == MSNH_F16;
    const std::string packPath = (weightCache && !_weightsPath.empty()) ? _weightsPath + (dtype == MSNH_F16 ? ".f16.pack" : ".f32.pack") : std::string();
    const std::string packLine = PackFile::headerLine(dtype, winograd);
    const uint64_t graphHash = packPath.empty() ? 0 : plan->structureHash() ^ (_graphTextHash * 0x9E3779B97F4A7C15ull);
    PackFile kept, fresh;
    t0 = Clock::now();
    const bool haveKept = !packPath.empty() && kept.open(packPath, packLine, _weightsHash, graphHash, plan->tensors.size());
    const float openMs = msSince(t0);

    t0 = Clock::now();
    if (dtype == MSNH_F16 && haveKept) plan->applyCalibration(kept.amax());
    else if (dtype == MSNH_F16)
    {
        // One float32 pass over a fixed pseudo-random U[0,1) input fixes the power-of-two scale of every
        // float16 tensor.  The float32 twin is lowered and optimised identically, so tensor ids line up.
        std::unique_ptr<Plan> cal = lowerNetwork(MSNH_F32);
        cal->fuseUpsample = plan->fuseUpsample;
        cal->fuse();
        cal->chainMaxPools();
        cal->aliasConcats();
        cal->place();
        setupYoloBuffers(*cal, _net->batch);
        cal->prepareWeights();
        float *host = _inputPinned.as<float>();
        uint32_t state = 0x9E3779B9u;
        for (int i = 0; i < _net->inputNum; ++i)
        {
            state = state * 1664525u + 1013904223u;
            host[i] = static_cast<float>(state >> 8) * (1.0f / 16777216.0f);
        }
        MSNH_DEV(msnh_hip_memcpy_h2d(_inputDev.ptr(), host, inBytes, _stream));
        if (cal->yoloCandCnt.ptr()) MSNH_DEV(msnh_hip_fill_zero(cal->yoloCandCnt.ptr(), cal->yoloCandCnt.bytes(), _stream));
        cal->runCalibration(_stream);
        plan->applyCalibration(cal->amaxOfTensors());
    }
    const float calMs = msSince(t0);
    t0 = Clock::now();
    plan->place();
    setupYoloBuffers(*plan, _net->batch);
    plan->preferWinograd = winograd;
    plan->sparseYolo = !_saveLayerOutput;         // layer dumps read the whole decoded tensors
    const bool writing = !packPath.empty() && !haveKept && fresh.create(packPath, packLine, _weightsHash, graphHash, plan->amaxOfTensors());
    plan->prepareWeights(haveKept ? &kept : nullptr, writing ? &fresh : nullptr);
    const char *packState = packPath.empty() ? "off" : "read";
    if (writing) packState = fresh.commit() ? "written" : "not writable";
    else if (haveKept && kept.stale())
    {
        // the file lacks a blob this plan asked for (the kernels were packed afresh): drop it, the next load writes a whole one
        std::remove(packPath.c_str());
        packState = "stale, removed";
    }
    const float packMs = msSince(t0);
    t0 = Clock::now();
    if (autoTune) plan->tuneConvs(_stream, (tuneCache && !_weightsPath.empty()) ? _weightsPath + (dtype == MSNH_F16 ? ".f16.tune" : ".f32.tune") : std::string());
    const float tuneMs = msSince(t0);
    {
        std::ostringstream os;
        os << "load: read+hash " << _readMs << " ms, lower " << lowerMs << " ms, pack file open " << openMs << " ms, calibrate " << calMs << " ms, place+pack+upload "
           << packMs << " ms, tune " << tuneMs << " ms; pack file " << packState;
        _loadDetail = os.str();
    }

    // hand every layer its slice of the op list
    for (size_t i = 0; i < _net->layers.size(); ++i)
    {
        BaseLayer *l = _net->layers[i];
        l->plan = plan.get();
        l->outTensor = plan->layerOut[i];
        size_t b = plan->ops.size(), e = 0;
        for (size_t k = 0; k < plan->ops.size(); ++k)
            if (plan->ops[k].layerIndex == static_cast<int>(i)) { b = std::min(b, k); e = std::max(e, k + 1); }
        if (e == 0) b = 0;
        l->opBegin = b; l->opEnd = e;
    }
    _net->plan = std::move(plan);
    _planReady = true;
}

// ---- run -------------------------------------------------------------------------------------------------------------
void NetBuilder::checkInput(size_t given) const
{
    if (BaseLayer::isPreviewMode) MSNH_THROW("Can not infer in preview mode !");
    if (_net->layers.empty()) MSNH_THROW("the network is not built");
    const size_t need = static_cast<size_t>(_net->inputNum);
    if (need != given) MSNH_THROW("input image size err. Needed :" + std::to_string(need) + " given :" + std::to_string(given));
    if (!_planReady) MSNH_THROW("weights are not loaded");
}

std::vector<float> NetBuilder::runClassify(std::vector<float>) { MSNH_THROW("Gpu mode , can not run with cpu"); }
std::vector<std::vector<YoloBox>> NetBuilder::runYolo(std::vector<float>) { MSNH_THROW("Gpu mode , can not run with cpu"); }

// Host floats -> pinned staging buffer -> device, in pieces: the workers copy piece k + 1 into the staging buffer while the
// DMA engine moves piece k (a batch of YOLOv3-608 is 35 MB: one thread's memcpy alone would take longer than the forward).
void NetBuilder::uploadInput(const float *img, size_t count)
{
    const size_t bytes = count * sizeof(float);
    const size_t piece = static_cast<size_t>(4) << 20, slice = static_cast<size_t>(512) << 10;
    const char *src = reinterpret_cast<const char *>(img);
    char *stage = static_cast<char *>(_inputPinned.ptr());
    TaskPool &pool = TaskPool::instance();
    for (size_t off = 0; off < bytes; off += piece)
    {
        const size_t len = std::min(piece, bytes - off);
        const int slices = static_cast<int>((len + slice - 1) / slice);
        pool.parallelFor(slices, [&](int i) {
            const size_t at = off + static_cast<size_t>(i) * slice;
            std::memcpy(stage + at, src + at, std::min(slice, off + len - at));
        });
        MSNH_DEV(msnh_hip_memcpy_h2d(_inputDev.as<char>() + off, stage + off, len, _stream));
    }
}

float *NetBuilder::deviceInputBuffer() { return _inputDev.as<float>(); }

void NetBuilder::setInputImageU8(int index, const unsigned char *rgbHwc, int width, int height, bool halfInit, bool shuffleRGB)
{
    setInputImage(index, rgbHwc, width, height, halfInit ? MSNH_PRE_PADDING_ZERO_HALF : MSNH_PRE_PADDING_ZERO, nullptr, nullptr, shuffleRGB);
}

void NetBuilder::setInputImage(int index, const unsigned char *rgbHwc, int width, int height, int preproc, const float *mean, const float *std, bool shuffleRGB)
{
    if (!_planReady) MSNH_THROW("weights are not loaded");
    if (rgbHwc == nullptr || width <= 0 || height <= 0) MSNH_THROW("img empty");
    if (_net->channels != 3) MSNH_THROW("the network does not take 3-channel images");
    if (index < 0 || index >= _net->batch) MSNH_THROW("image index outside the batch");
    if (preproc == MSNH_PRE_TRANSFORMED && (mean == nullptr || std == nullptr)) MSNH_THROW("mean or std can't be null");
    const size_t bytes = static_cast<size_t>(width) * height * 3;
    // the pinned staging buffer is reused by the next call: wait for the previous upload before overwriting it
    MSNH_DEV(msnh_hip_stream_sync(_stream));
    _imagePinned.reserve(bytes);
    if (_imageDev.bytes() < bytes) _imageDev.alloc(bytes);
    std::memcpy(_imagePinned.ptr(), rgbHwc, bytes);
    MSNH_DEV(msnh_hip_memcpy_h2d(_imageDev.ptr(), _imagePinned.ptr(), bytes, _stream));
    float *dst = _inputDev.as<float>() + static_cast<size_t>(index) * 3 * _net->height * _net->width;
    MSNH_DEV(msnh_hip_image_u8_to_input(static_cast<const unsigned char *>(_imageDev.ptr()), width, height, _net->width, _net->height, preproc, mean, std,
                                        shuffleRGB ? 1 : 0, dst, _stream));
}

static std::vector<float> yoloLayerDump(Plan &plan, const YoloLayer *yl, const PlanOp &op, int batch, msnh_stream_t s)
{
    // decoded rows [cell][5+classes] of this head -> the reference's NCHW [anchor*(5+classes)+m][pixel] order
    const int per = 5 + op.classes;
    const int hw = yl->getOutHeight() * yl->getOutWidth();
    std::vector<float> all(static_cast<size_t>(plan.yoloCells) * per * batch);
    MSNH_DEV(msnh_hip_memcpy_d2h(all.data(), plan.yoloDecoded.ptr(), all.size() * sizeof(float), s));
    MSNH_DEV(msnh_hip_stream_sync(s));
    std::vector<float> out(static_cast<size_t>(batch) * 3 * per * hw);
    for (int b = 0; b < batch; ++b)
        for (int a = 0; a < 3; ++a)
            for (int p = 0; p < hw; ++p)
                for (int m = 0; m < per; ++m)
                    out[((static_cast<size_t>(b) * 3 + a) * per + m) * hw + p] =
                        all[(static_cast<size_t>(b) * plan.yoloCells + op.cellBase + static_cast<size_t>(a) * hw + p) * per + m];
    return out;
}

void NetBuilder::runLayersEager()
{
    Plan &plan = *_net->plan;
    if (plan.yoloCandCnt.ptr()) MSNH_DEV(msnh_hip_fill_zero(plan.yoloCandCnt.ptr(), plan.yoloCandCnt.bytes(), _stream));
    _layerOutputs.assign(_net->layers.size(), std::vector<float>());
    msnh_event_t e0 = nullptr, e1 = nullptr;
    MSNH_DEV(msnh_hip_event_create(&e0));
    MSNH_DEV(msnh_hip_event_create(&e1));
    for (size_t i = 0; i < _net->layers.size(); ++i)
    {
        BaseLayer *l = _net->layers[i];
        MSNH_DEV(msnh_hip_event_record(e0, _stream));
        l->forwardGPU(*_netState);
        MSNH_DEV(msnh_hip_event_record(e1, _stream));
        MSNH_DEV(msnh_hip_event_sync(e1));
        float ms = 0.f;
        MSNH_DEV(msnh_hip_event_elapsed_ms(e0, e1, &ms));
        l->setForwardTime(ms);
        if (!_saveLayerOutput) continue;
        if (l->type() == LayerType::YOLO)
        {
            const YoloLayer *yl = static_cast<const YoloLayer *>(l);
            _layerOutputs[i] = yoloLayerDump(plan, yl, plan.ops[yl->decodeOp], _net->batch, _stream);
        }
        else if (l->type() != LayerType::YOLO_OUT)
        {
            plan.exportTensor(plan.layerOut[i], _layerOutputs[i], _stream);
        }
        if (_writeDumpFiles)
        {
            std::ofstream f(std::to_string(i) + "gpu.txt");
            for (float v : _layerOutputs[i]) f << v << "\n";
        }
    }
    msnh_hip_event_destroy(e0);
    msnh_hip_event_destroy(e1);
}

void NetBuilder::enqueueForward(const float *deviceInput)
{
    if (!_planReady) MSNH_THROW("weights are not loaded");
    Plan &plan = *_net->plan;
    YoloOutLayer *yout = _net->layers.back()->type() == LayerType::YOLO_OUT ? static_cast<YoloOutLayer *>(_net->layers.back()) : nullptr;
    if (yout && _inFlight >= 2) MSNH_THROW("two forwards are already in flight: fetch a result first");
    if (deviceInput != nullptr && deviceInput != _inputDev.as<float>())
        MSNH_DEV(msnh_hip_memcpy_d2d(_inputDev.ptr(), deviceInput, sizeof(float) * static_cast<size_t>(_net->inputNum), _stream));
    if (yout && plan.sparseYolo && plan.yoloKeepDecoded != YoloOutLayer::keepClassScores)
    {
        // the full decoded rows are only written for YoloBox::classesVal; the recorded launches carry the choice
        plan.yoloKeepDecoded = YoloOutLayer::keepClassScores;
        if (_graph) { msnh_hip_graph_destroy(_graph); _graph = nullptr; }
    }
    static const bool eager = std::getenv("MSNH_EAGER") != nullptr;
    if (eager)
    {
        if (plan.yoloCandCnt.ptr()) MSNH_DEV(msnh_hip_fill_zero(plan.yoloCandCnt.ptr(), plan.yoloCandCnt.bytes(), _stream));
        plan.runAll(_stream);
        if (yout) yout->enqueueGather(_stream);
    }
    else if (_graph == nullptr)
    {
        // Record the whole forward once; later calls replay it with a single launch.
        MSNH_DEV(msnh_hip_graph_begin(_stream));
        try
        {
            if (plan.yoloCandCnt.ptr()) MSNH_DEV(msnh_hip_fill_zero(plan.yoloCandCnt.ptr(), plan.yoloCandCnt.bytes(), _stream));
            plan.runAll(_stream);
            if (yout) yout->enqueueGather(_stream);
        }
        catch (...)
        {
            msnh_graph_t junk = nullptr;
            msnh_hip_graph_end(_stream, &junk);
            if (junk) msnh_hip_graph_destroy(junk);
            throw;
        }
        MSNH_DEV(msnh_hip_graph_end(_stream, &_graph));
    }
    if (!eager) MSNH_DEV(msnh_hip_graph_launch(_graph, _stream));
    if (yout)
    {
        // results leave the device right behind the forward, so the next forward can start while the host sorts
        yout->enqueueCopyBack(_stream, _nextSlot);
        _nextSlot ^= 1;
        ++_inFlight;
    }
}

void NetBuilder::sync() { MSNH_DEV(msnh_hip_stream_sync(_stream)); }

std::vector<float> NetBuilder::fetchClassify()
{
    Plan &plan = *_net->plan;
    std::vector<float> out;
    plan.exportTensor(plan.layerOut.back(), out, _stream);
    return out;
}

std::vector<std::vector<YoloBox>> NetBuilder::fetchYolo()
{
    BaseLayer *last = _net->layers.back();
    if (last->type() != LayerType::YOLO_OUT) MSNH_THROW("not a yolo net");
    YoloOutLayer *yout = static_cast<YoloOutLayer *>(last);
    if (_inFlight <= 0)
    {
        if (yout->finalOut.empty()) MSNH_THROW("no forward in flight");
        return yout->finalOut;                                  // nothing new: the last result again
    }
    const int slot = (_nextSlot + 2 - _inFlight) & 1;          // oldest outstanding
    yout->finish(slot);
    --_inFlight;
    return yout->finalOut;
}

std::vector<float> NetBuilder::yoloHeadLogits(int head)
{
    if (!_planReady) MSNH_THROW("weights are not loaded");
    if (_inFlight > 0) MSNH_THROW("fetch the outstanding results first");
    Plan &plan = *_net->plan;
    std::vector<size_t> heads = plan.yoloHeadOps;
    if (heads.empty())
    {
        // heads decoded one by one: their inputs are only kept to the end of the forward while layer dumps pin them
        if (!_saveLayerOutput) MSNH_THROW("the head tensors of this plan do not outlive the forward (run with layer dumps on)");
        for (size_t i = 0; i < plan.ops.size(); ++i)
            if (plan.ops[i].kind == PlanOp::YOLO_DECODE && !plan.ops[i].dead) heads.push_back(i);
        std::sort(heads.begin(), heads.end(), [&plan](size_t a, size_t b) { return plan.ops[a].cellBase < plan.ops[b].cellBase; });
    }
    if (head < 0 || static_cast<size_t>(head) >= heads.size()) MSNH_THROW("no such detection head");
    std::vector<float> out;
    plan.exportTensor(plan.ops[heads[static_cast<size_t>(head)]].in0, out, _stream);
    return out;
}

std::vector<float> NetBuilder::yoloLastCandidates(int image)
{
    BaseLayer *last = _net->layers.empty() ? nullptr : _net->layers.back();
    if (last == nullptr || last->type() != LayerType::YOLO_OUT) MSNH_THROW("not a yolo net");
    return static_cast<YoloOutLayer *>(last)->lastCandidateRows(image);
}

std::vector<float> NetBuilder::runClassifyGPU(std::vector<float> img) { return runClassifyGPU(img.data(), img.size()); }
std::vector<std::vector<YoloBox>> NetBuilder::runYoloGPU(std::vector<float> img) { return runYoloGPU(img.data(), img.size()); }

std::vector<float> NetBuilder::runClassifyGPU(const float *img, size_t count)
{
    checkInput(count);
    if (img == nullptr) MSNH_THROW("input image is NULL");
    auto st = TimeUtil::startRecord();
    uploadInput(img, count);
    std::vector<float> out;
    if (_saveLayerOutput)
    {
        runLayersEager();
        _net->plan->exportTensor(_net->plan->layerOut.back(), out, _stream);
    }
    else
    {
        enqueueForward(nullptr);
        out = fetchClassify();
    }
    _gpuInferenceTime = TimeUtil::getElapsedTime(st);
    return out;
}

std::vector<std::vector<YoloBox>> NetBuilder::runYoloGPU(const float *img, size_t count)
{
    checkInput(count);
    if (img == nullptr) MSNH_THROW("input image is NULL");
    if (_net->layers.back()->type() != LayerType::YOLO_OUT) MSNH_THROW("not a yolo net");
    auto st = TimeUtil::startRecord();
    uploadInput(img, count);
    std::vector<std::vector<YoloBox>> out;
    if (_saveLayerOutput)
    {
        runLayersEager();
        out = static_cast<YoloOutLayer *>(_net->layers.back())->finalOut;
    }
    else
    {
        enqueueForward(nullptr);
        out = fetchYolo();
    }
    _gpuInferenceTime = TimeUtil::getElapsedTime(st);
    return out;
}

float NetBuilder::fp16Headroom(const std::vector<float> &img)
{
    checkInput(img.size());
    if (_inFlight > 0) MSNH_THROW("fetch the outstanding results first");
    uploadInput(img.data(), img.size());
    return _net->plan->fp16Headroom(_stream);
}

// ---- getters ---------------------------------------------------------------------------------------------------------
Point2I NetBuilder::getInputSize()
{
    if (_parser->params.empty()) MSNH_THROW("net param is empty");
    if (_parser->params[0]->type != LayerType::CONFIG) MSNH_THROW("net param error");
    NetConfigParams *cfg = static_cast<NetConfigParams *>(_parser->params[0]);
    return Point2I(cfg->width, cfg->height);
}

int NetBuilder::getInputChannel()
{
    if (_parser->params.empty()) MSNH_THROW("net param is empty");
    return static_cast<NetConfigParams *>(_parser->params[0])->channels;
}

int NetBuilder::getBatch() const { return _net->batch; }
bool NetBuilder::lastNmsOnDevice() const
{
    BaseLayer *last = _net->layers.empty() ? nullptr : _net->layers.back();
    return last && last->type() == LayerType::YOLO_OUT && static_cast<YoloOutLayer *>(last)->lastOnDevice;
}

float NetBuilder::getInferenceTime()
{
    float t = 0.f;
    for (BaseLayer *l : _net->layers) t += l->getForwardTime();
    return t;
}

static std::string index3(size_t i)
{
    return i < 10 ? "00" + std::to_string(i) : (i < 100 ? "0" + std::to_string(i) : std::to_string(i));
}

std::string NetBuilder::getLayerDetail()
{
    std::string d;
    for (size_t i = 0; i < _net->layers.size(); ++i)
    {
        d += "────────────────────────────────  " + index3(i) + " ─────────────────────────────────\n";
        d += _net->layers[i]->getLayerDetail() + "weights : " + std::to_string(_net->layers[i]->getNumWeights()) + "\n\n";
    }
    return d;
}

std::string NetBuilder::getTimeDetail()
{
    const float total = getInferenceTime();
    std::string d = "LAYER            INDEX       TIME         LAYER_t/TOTAL_t\r\n=========================================================\n";
    for (size_t i = 0; i < _net->layers.size(); ++i)
    {
        const float t = _net->layers[i]->getForwardTime();
        d += _net->layers[i]->getLayerName() + " : " + index3(i) + "     " + std::to_string(t).substr(0, 6) + " ms         " +
             std::to_string(static_cast<int>(t / total * 1000) / 10.f).substr(0, 4) + "%\n";
    }
    d += "=========================================================\n";
    if (!_net->layers.empty() && _net->layers.back()->type() == LayerType::YOLO_OUT) d += static_cast<YoloOutLayer *>(_net->layers.back())->placementDetail();
    d += "Msnhnet inference time : " + std::to_string(total) + " ms";
    return d;
}

float NetBuilder::getGpuInferenceTime() const { return _gpuInferenceTime; }
Network *NetBuilder::getNet() const { return _net; }
int NetBuilder::getLastLayerOutWidth() const { return _lastLayerOutWidth; }
int NetBuilder::getLastLayerOutHeight() const { return _lastLayerOutHeight; }
int NetBuilder::getLastLayerOutChannel() const { return _lastLayerOutChannel; }
size_t NetBuilder::getLastLayerOutNum() const { return _lastLayerOutNum; }
bool NetBuilder::getSaveLayerWeights() const { return _saveLayerWeights; }
void NetBuilder::setSaveLayerWeights(bool v) { _saveLayerWeights = v; }

void NetBuilder::setSaveLayerOutput(bool v)
{
    if (v == _saveLayerOutput) return;
    _saveLayerOutput = v;
    // dumps need every layer output as a real tensor: re-plan if a plan already exists
    if (_planReady) finalizePlan();
}

static double opBytes(const Plan &plan, const PlanOp &op)
{
    // what the launch must move at least: its input, its output, a fused residual, its weights
    const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
    const PlanTensor &out = plan.tensors[static_cast<size_t>(op.out)];
    double oe = static_cast<double>(out.elems()) * (out.dtype == MSNH_F16 ? 2 : 4);
    for (int nx = op.chainNext; nx >= 0; nx = plan.ops[static_cast<size_t>(nx)].chainNext) oe += static_cast<double>(out.elems()) * (out.dtype == MSNH_F16 ? 2 : 4);   // one launch, every pool's result
    if (op.stemTail >= 0)
    {
        const PlanOp &b = plan.ops[static_cast<size_t>(op.stemTail)];
        oe += static_cast<double>(plan.tensors[static_cast<size_t>(b.out)].elems()) * 2 + static_cast<double>(op.wDev3.bytes());
    }
    if (op.algo == MSNH_CONV_IGEMM_TAIL && op.tail >= 0)
    {
        // ... and the 1x1 convolution computed by the same launch: its result and its filters
        const PlanOp &b = plan.ops[static_cast<size_t>(op.tail)];
        oe += static_cast<double>(plan.tensors[static_cast<size_t>(b.out)].elems()) * 2 + static_cast<double>(b.wDev.bytes());
    }
    return static_cast<double>(in.elems()) * (in.dtype == MSNH_F16 ? 2 : 4) + oe + (op.in1 >= 0 ? static_cast<double>(out.elems()) * (out.dtype == MSNH_F16 ? 2 : 4) : 0.0) +
           static_cast<double>(op.wDev.bytes());
}

float NetBuilder::profileOps(int kind, int reps, int *launches, double *flops, double *bytes)
{
    if (!_planReady) MSNH_THROW("weights are not loaded");
    Plan &plan = *_net->plan;
    msnh_event_t e0 = nullptr, e1 = nullptr;
    MSNH_DEV(msnh_hip_event_create(&e0));
    MSNH_DEV(msnh_hip_event_create(&e1));
    int n = 0;
    double f = 0, by = 0;
    MSNH_DEV(msnh_hip_event_record(e0, _stream));
    for (int r = 0; r < reps; ++r)
        for (size_t i = 0; i < plan.ops.size(); ++i)
        {
            const PlanOp &op = plan.ops[i];
            // kind: a PlanOp::Kind, -1 for every launch, or 1000 + a convolution algorithm (MSNH_CONV_*)
            if (op.dead || op.chainHead >= 0) continue;
            if (kind >= 1000 ? (op.kind != PlanOp::CONV || op.algo != kind - 1000) : (kind >= 0 && static_cast<int>(op.kind) != kind)) continue;
            plan.run(i, i + 1, _stream);
            ++n;
            f += op.flops;
            by += opBytes(plan, op);
        }
    MSNH_DEV(msnh_hip_event_record(e1, _stream));
    MSNH_DEV(msnh_hip_event_sync(e1));
    float ms = 0.f;
    MSNH_DEV(msnh_hip_event_elapsed_ms(e0, e1, &ms));
    msnh_hip_event_destroy(e0);
    msnh_hip_event_destroy(e1);
    if (launches) *launches = n;
    if (flops) *flops = f;
    if (bytes) *bytes = by;
    return ms;
}

std::string NetBuilder::profileEachOp(int reps, std::vector<double> *values)
{
    if (!_planReady) MSNH_THROW("weights are not loaded");
    Plan &plan = *_net->plan;
    static const char *kinds[] = {"conv", "affine", "add", "copy", "maxpool", "avgpool", "upsample", "connected", "input_cast", "yolo_decode", "pad", "slice", "bilinear", "softmax", "col2im"};
    static const char *algos[] = {"auto", "direct", "igemm", "depthwise", "winograd", "stem", "igemm_splitk", "pointwise", "stem+down", "winograd_fused", "mbconv", "igemm+1x1"};
    msnh_event_t e0 = nullptr, e1 = nullptr;
    MSNH_DEV(msnh_hip_event_create(&e0));
    MSNH_DEV(msnh_hip_event_create(&e1));
    std::ostringstream os;
    double totalUs = 0;
    for (size_t i = 0; i < plan.ops.size(); ++i)
    {
        const PlanOp &op = plan.ops[i];
        if (op.dead || op.chainHead >= 0) continue;
        plan.run(i, i + 1, _stream);
        const bool yolo = op.kind == PlanOp::YOLO_DECODE && plan.yoloCandCnt.ptr();
        MSNH_DEV(msnh_hip_event_record(e0, _stream));
        for (int r = 0; r < reps; ++r)
        {
            // (a head appends to the candidate list: start every repetition from an empty one, as a forward does)
            if (yolo) MSNH_DEV(msnh_hip_fill_zero(plan.yoloCandCnt.ptr(), plan.yoloCandCnt.bytes(), _stream));
            plan.run(i, i + 1, _stream);
        }
        MSNH_DEV(msnh_hip_event_record(e1, _stream));
        MSNH_DEV(msnh_hip_event_sync(e1));
        float ms = 0.f;
        MSNH_DEV(msnh_hip_event_elapsed_ms(e0, e1, &ms));
        const double us = ms * 1e3 / reps;
        totalUs += us;
        if (values)
        {
            const double row[8] = {static_cast<double>(op.kind), static_cast<double>(op.algo), static_cast<double>(op.layerIndex), static_cast<double>(op.tile),
                                   op.flops, opBytes(plan, op), us, static_cast<double>(op.ksize * 100 + op.stride)};
            values->insert(values->end(), row, row + 8);
        }
        const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
        const PlanTensor &out = plan.tensors[static_cast<size_t>(op.out)];
        const double bytes = static_cast<double>(in.elems()) * (in.dtype == MSNH_F16 ? 2 : 4) + static_cast<double>(out.elems()) * (out.dtype == MSNH_F16 ? 2 : 4) +
                             (op.in1 >= 0 ? static_cast<double>(out.elems()) * (out.dtype == MSNH_F16 ? 2 : 4) : 0.0);
        char line[320];
        snprintf(line, sizeof(line), "L%-3d %-11s %-9s t%-2d k%d s%d g%-4d %4dx%4dx%4dx%4d -> %4dx%4dx%4d %s%s %9.2f us %8.2f TF/s %8.1f GB/s\n", op.layerIndex,
                 kinds[op.kind], (op.kind == PlanOp::CONV || op.algo != MSNH_CONV_AUTO) ? algos[op.algo] : "-", op.tile, op.ksize, op.stride, op.groups, in.n, in.h, in.w, in.c, out.h, out.w,
                 out.c, out.dtype == MSNH_F16 ? "f16" : "f32", op.in1 >= 0 ? "+res" : "    ", us, op.flops / us * 1e-6, bytes / us * 1e-3);
        os << line;
    }
    os << "total " << totalUs << " us over " << plan.liveOps() << " launches\n";
    msnh_hip_event_destroy(e0);
    msnh_hip_event_destroy(e1);
    return os.str();
}

std::string NetBuilder::getLoadDetail() const { return _loadDetail; }
std::string NetBuilder::getPlanDetail() const { return _net->plan ? _net->plan->describe() : std::string(); }
double NetBuilder::getConvFlops() const { return _net->plan ? _net->plan->totalConvFlops() : 0.0; }
}
