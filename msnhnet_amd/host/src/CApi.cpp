// C ABI of the host library (include/msnhnet_c.h): the reference facade over one global NetBuilder plus the
// handle-based variant.  Every entry point catches all exceptions; none of them lets one cross the boundary.
#include "msnhnet_c.h"
#include <algorithm>
#include <cstring>
#include <memory>
#include <string>
#include "Msnhnet/net/MsnhNetBuilder.h"
#include "Msnhnet/net/MsnhNetGroup.h"
#include "Msnhnet/layers/MsnhLayers.h"

using namespace Msnhnet;

namespace
{
thread_local std::string g_lastError;
std::unique_ptr<NetBuilder> g_net;

char *keepError(const std::exception &e)
{
    g_lastError = e.what();
    return const_cast<char *>(g_lastError.c_str());
}

template <typename F> int guarded(F &&f)
{
    try { f(); return 0; }
    catch (const std::exception &e) { keepError(e); return 1; }
    catch (...) { g_lastError = "unknown error"; return 1; }
}

template <typename F> int refStyle(char **msg, F &&f)
{
    try { f(); return 1; }
    catch (const std::exception &e) { char *m = keepError(e); if (msg) *msg = m; return -1; }
    catch (...) { g_lastError = "unknown error"; if (msg) *msg = const_cast<char *>(g_lastError.c_str()); return -1; }
}

NetBuilder &nb(msnhnet_t h)
{
    if (h == nullptr) MSNH_THROW("net handle is NULL");
    return *static_cast<NetBuilder *>(h);
}

long long copyText(const std::string &s, char *dst, long long cap)
{
    if (dst && cap > 0)
    {
        const long long n = std::min<long long>(static_cast<long long>(s.size()), cap - 1);
        std::memcpy(dst, s.data(), static_cast<size_t>(n));
        dst[n] = 0;
    }
    return static_cast<long long>(s.size());
}

void packBoxes(const std::vector<std::vector<YoloBox>> &all, int *counts, float *boxes, long long cap, long long *total)
{
    long long w = 0, sum = 0;
    for (size_t b = 0; b < all.size(); ++b)
    {
        if (counts) counts[b] = static_cast<int>(all[b].size());
        sum += static_cast<long long>(all[b].size());
        for (const YoloBox &q : all[b])
        {
            if (boxes && w < cap)
            {
                float *o = boxes + 7 * w;
                o[0] = q.xywhBox.x; o[1] = q.xywhBox.y; o[2] = q.xywhBox.w; o[3] = q.xywhBox.h;
                o[4] = q.conf; o[5] = q.bestClsConf; o[6] = static_cast<float>(q.bestClsIdx);
            }
            ++w;
        }
    }
    if (total) *total = sum;
}
}

extern "C" {

// ---- part 1 -----------------------------------------------------------------------------------------------------------
int initMsnhnet(void)
{
    try { g_net.reset(new NetBuilder()); return 1; }
    catch (const std::exception &e) { keepError(e); return -1; }
}

int buildMsnhnet(char **msg, const char *msnhnet, const char *msnhbin, int useFp16, int useCudaOnly)
{
    return refStyle(msg, [&] {
        if (!g_net) MSNH_THROW("initMsnhnet was not called");
        if (!msnhnet || !msnhbin) MSNH_THROW("path is NULL");
        NetBuilder::setUseFp16(useFp16 != 0);
        NetBuilder::setForceUseCuda(useCudaOnly != 0);
        g_net->buildNetFromMsnhNet(msnhnet);
        g_net->loadWeightsFromMsnhBin(msnhbin);
    });
}

int runClassifyNoPred(char **msg, const float *data, const int len, int *bestIndex, int runGPU)
{
    return refStyle(msg, [&] {
        if (!g_net) MSNH_THROW("initMsnhnet was not called");
        if (!data || !bestIndex || len <= 0) MSNH_THROW("bad argument");
        std::vector<float> img(data, data + len);
        const std::vector<float> out = runGPU ? g_net->runClassifyGPU(img) : g_net->runClassify(img);
        const size_t per = g_net->getLastLayerOutNum();
        *bestIndex = static_cast<int>(std::distance(out.begin(), std::max_element(out.begin(), out.begin() + static_cast<long long>(per))));
    });
}

int runYoloNoPred(char **msg, const float *data, const int len, BBoxContainer *bboxContainer, int *detectedNum, int runGPU)
{
    return refStyle(msg, [&] {
        if (!g_net) MSNH_THROW("initMsnhnet was not called");
        if (!data || !bboxContainer || !detectedNum || len <= 0) MSNH_THROW("bad argument");
        std::vector<float> img(data, data + len);
        const std::vector<std::vector<YoloBox>> out = runGPU ? g_net->runYoloGPU(img) : g_net->runYolo(img);
        const std::vector<YoloBox> &b0 = out.at(0);
        const size_t n = std::min<size_t>(b0.size(), MSNHNET_MAX_BBOX);
        for (size_t i = 0; i < n; ++i)
        {
            BBox &o = bboxContainer->boxes[i];
            o.x = b0[i].xywhBox.x; o.y = b0[i].xywhBox.y; o.w = b0[i].xywhBox.w; o.h = b0[i].xywhBox.h;
            o.conf = b0[i].conf; o.bestClsConf = b0[i].bestClsConf; o.bestClsIdx = static_cast<uint32_t>(b0[i].bestClsIdx); o.angle = b0[i].angle;
        }
        *detectedNum = static_cast<int>(n);
    });
}

// The byte-image entry points: pre-processing on the device (msnh_hip_image_u8_to_input), then the forward on what it wrote.
static int preprocOf(int preDataType, int channel)
{
    if (channel != 1 && channel != 3) MSNH_THROW("channel must be 1 or 3");
    if (channel == 1 && preDataType != PRE_DATA_FC32_C1) MSNH_THROW("channel 1 must preprocess with F32_C1");
    if (channel == 3 && preDataType == PRE_DATA_FC32_C1) MSNH_THROW("channel 1 can't preprocess with F32_C1");
    // (the reference's own gray-image loop reads the resized image with the extent of the original one,
    //  src/utils/MsnhCVUtil.cpp:47-82; this build takes 3-channel images only)
    if (channel == 1) MSNH_THROW("1-channel images are outside the convolutional path this build implements");
    switch (preDataType)
    {
    case PRE_DATA_FC32_C3:          return MSNH_PRE_F32C3;
    case PRE_DATA_GOOGLENET_FC3:    return MSNH_PRE_GOOGLENET;
    case PRE_DATA_PADDING_ZERO_FC3: return MSNH_PRE_PADDING_ZERO;
    case PRE_DATA_TRANSFORMED_FC3:  return MSNH_PRE_TRANSFORMED;
    case PRE_DATA_CAFFE_FC3:        return MSNH_PRE_CAFFE;
    default: break;
    }
    MSNH_THROW("preDataType can't be none");
}

// Whether the network sees the first and third channel of the caller's image exchanged.  The reference's facade (its build without
// OpenCV) exchanges them itself when swapRGB == 0 (src/c_api/MsnhnetLib.cpp:562-565, :771-774) and then calls the CVUtil function
// with its default needShuffleRGB, which exchanges them once more for every variant but the letterbox
// (include/Msnhnet/utils/MsnhCVUtil.h:23-38: true for getImgDataF32C3 / getGoogLenetF32C3 / getTransformedF32C3 / getCaffeModeF32C3,
// false for getPaddingZeroF32C3).  Net effect: exchanged when swapRGB != 0, except for the letterbox, where it is exchanged when
// swapRGB == 0.
static bool facadeShuffle(int kind, int swapRGB) { return kind == MSNH_PRE_PADDING_ZERO ? swapRGB == 0 : swapRGB != 0; }

int runClassifyList(char **msg, unsigned char *imageData, const int width, const int height, const int channel, int *bestIndex, int preDataType,
                    const int swapRGB, int runGPU, const float *mean, const float *std)
{
    return refStyle(msg, [&] {
        if (!g_net) MSNH_THROW("initMsnhnet was not called");
        if (!imageData || !bestIndex) MSNH_THROW("bad argument");
        const int kind = preprocOf(preDataType, channel);
        if (kind == MSNH_PRE_TRANSFORMED && (mean == nullptr || std == nullptr)) MSNH_THROW("mean or std can't be null");
        if (!runGPU) g_net->runClassify(std::vector<float>());           // throws: this build has no CPU path
        if (g_net->getBatch() != 1) MSNH_THROW("runClassifyList takes one image: build the graph with batch 1");
        g_net->setInputImage(0, imageData, width, height, kind, mean, std, facadeShuffle(kind, swapRGB));
        g_net->enqueueForward(nullptr);
        const std::vector<float> out = g_net->fetchClassify();
        *bestIndex = static_cast<int>(std::distance(out.begin(), std::max_element(out.begin(), out.end())));
    });
}

int runYoloList(char **msg, unsigned char *imageData, const int width, const int height, const int channel, BBoxContainer *bboxContainer,
                int *detectedNum, const int swapRGB, const int runGPU)
{
    return refStyle(msg, [&] {
        if (!g_net) MSNH_THROW("initMsnhnet was not called");
        if (!imageData || !bboxContainer || !detectedNum) MSNH_THROW("bad argument");
        if (channel != 1 && channel != 3) MSNH_THROW("channel must be 1 or 3");
        if (channel == 1) MSNH_THROW("1-channel images are outside the convolutional path this build implements");
        if (!runGPU) g_net->runYolo(std::vector<float>());               // throws: this build has no CPU path
        if (g_net->getBatch() != 1) MSNH_THROW("runYoloList takes one image: build the graph with batch 1");
        g_net->setInputImage(0, imageData, width, height, MSNH_PRE_PADDING_ZERO, nullptr, nullptr, facadeShuffle(MSNH_PRE_PADDING_ZERO, swapRGB));
        g_net->enqueueForward(nullptr);
        const std::vector<std::vector<YoloBox>> out = g_net->fetchYolo();
        const std::vector<YoloBox> &b0 = out.at(0);
        if (b0.size() > MSNHNET_MAX_BBOX) MSNH_THROW("BBox buffer is not enough, please change MaxBBoxNum and rebuild");
        *detectedNum = static_cast<int>(b0.size());
        for (size_t i = 0; i < b0.size(); ++i)
        {
            BBox &o = bboxContainer->boxes[i];
            o.x = b0[i].xywhBox.x; o.y = b0[i].xywhBox.y; o.w = b0[i].xywhBox.w; o.h = b0[i].xywhBox.h;
            o.conf = b0[i].conf; o.bestClsConf = b0[i].bestClsConf; o.bestClsIdx = static_cast<uint32_t>(b0[i].bestClsIdx); o.angle = b0[i].angle;
        }
    });
}

int dispose(void) { g_net.reset(); return 1; }

int withGPU(int *GPU)
{
    if (!GPU) return -1;
    int count = 0;
    msnh_hip_device_count(&count);
    *GPU = count > 0 ? 1 : 0;
    return 1;
}

int withCUDNN(int *CUDNN)
{
    if (!CUDNN) return -1;
    *CUDNN = 0;
    return 1;
}

int getCpuForwardTime(float *time)
{
    if (!time || !g_net) return -1;
    *time = g_net->getInferenceTime();
    return 1;
}

int getGpuForwardTime(float *time)
{
    if (!time || !g_net) return -1;
    *time = g_net->getGpuInferenceTime();
    return 1;
}

int getInputDim(int *width, int *heigth, int *channel)
{
    return refStyle(nullptr, [&] {
        if (!g_net || !width || !heigth || !channel) MSNH_THROW("bad argument");
        const Point2I p = g_net->getInputSize();
        *width = p.x; *heigth = p.y; *channel = g_net->getInputChannel();
    });
}

// ---- part 2 -----------------------------------------------------------------------------------------------------------
const char *msnhnet_last_error(void) { return g_lastError.c_str(); }

int msnhnet_create(msnhnet_t *net)
{
    return guarded([&] { if (!net) MSNH_THROW("net pointer is NULL"); *net = new NetBuilder(); });
}

int msnhnet_destroy(msnhnet_t net)
{
    return guarded([&] { delete static_cast<NetBuilder *>(net); });
}

int msnhnet_set_use_fp16(int on) { return guarded([&] { NetBuilder::setUseFp16(on != 0); }); }
int msnhnet_set_use_winograd(int on) { return guarded([&] { NetBuilder::setUseWinograd(on != 0); }); }
int msnhnet_set_device_nms(int mode) { return guarded([&] { NetBuilder::setDeviceNms(mode); }); }
int msnhnet_set_tune_cache(int on) { return guarded([&] { NetBuilder::setTuneCache(on != 0); }); }
int msnhnet_set_weight_cache(int on) { return guarded([&] { NetBuilder::setWeightCache(on != 0); }); }
int msnhnet_set_keep_class_scores(int on) { return guarded([&] { NetBuilder::setKeepClassScores(on != 0); }); }
int msnhnet_set_save_layer_output(msnhnet_t net, int on) { return guarded([&] { nb(net).setSaveLayerOutput(on != 0); }); }
int msnhnet_build(msnhnet_t net, const char *path) { return guarded([&] { if (!path) MSNH_THROW("path is NULL"); nb(net).buildNetFromMsnhNet(path); }); }
int msnhnet_load(msnhnet_t net, const char *path) { return guarded([&] { if (!path) MSNH_THROW("path is NULL"); nb(net).loadWeightsFromMsnhBin(path); }); }

int msnhnet_load_from_memory(msnhnet_t net, const float *weights, size_t count)
{
    return guarded([&] {
        if (!weights && count) MSNH_THROW("weights is NULL");
        nb(net).loadWeightsFromVector(std::vector<float>(weights, weights + count));
    });
}

int msnhnet_input_dims(msnhnet_t net, int *batch, int *channels, int *height, int *width)
{
    return guarded([&] {
        Network *n = nb(net).getNet();
        if (batch) *batch = n->batch;
        if (channels) *channels = n->channels;
        if (height) *height = n->height;
        if (width) *width = n->width;
    });
}

int msnhnet_num_layers(msnhnet_t net)
{
    int n = -1;
    guarded([&] { n = static_cast<int>(nb(net).getNet()->layers.size()); });
    return n;
}

int msnhnet_layer_info(msnhnet_t net, int layer, long long *info, char *name, int name_cap)
{
    return guarded([&] {
        Network *n = nb(net).getNet();
        if (layer < 0 || static_cast<size_t>(layer) >= n->layers.size() || !info) MSNH_THROW("layer index out of range");
        const BaseLayer *l = n->layers[static_cast<size_t>(layer)];
        info[0] = static_cast<long long>(l->type()); info[1] = l->getOutHeight(); info[2] = l->getOutWidth(); info[3] = l->getOutChannel();
        info[4] = l->getOutputNum(); info[5] = l->getInputNum(); info[6] = static_cast<long long>(l->getNumWeights()); info[7] = l->getMemReUse();
        info[8] = l->getBatch(); info[9] = static_cast<long long>(l->getActivation());
        copyText(l->getLayerName(), name, name_cap);
    });
}

long long msnhnet_layer_detail(msnhnet_t net, char *dst, long long cap)
{
    long long n = -1;
    guarded([&] { n = copyText(nb(net).getLayerDetail(), dst, cap); });
    return n;
}

long long msnhnet_plan_detail(msnhnet_t net, char *dst, long long cap)
{
    long long n = -1;
    guarded([&] { n = copyText(nb(net).getPlanDetail(), dst, cap); });
    return n;
}

long long msnhnet_load_detail(msnhnet_t net, char *dst, long long cap)
{
    long long n = -1;
    guarded([&] { n = copyText(nb(net).getLoadDetail(), dst, cap); });
    return n;
}

long long msnhnet_time_detail(msnhnet_t net, char *dst, long long cap)
{
    long long n = -1;
    guarded([&] { n = copyText(nb(net).getTimeDetail(), dst, cap); });
    return n;
}

long long msnhnet_weight_layout(msnhnet_t net, long long *parts, long long cap)
{
    long long n = -1;
    guarded([&] {
        std::vector<long long> all;
        for (const BaseLayer *l : nb(net).getNet()->layers) l->weightLayout(all);
        n = static_cast<long long>(all.size() / 3);
        if (parts && cap > 0) std::memcpy(parts, all.data(), sizeof(long long) * static_cast<size_t>(std::min<long long>(cap, n) * 3));
    });
    return n;
}

double msnhnet_conv_flops(msnhnet_t net)
{
    double f = 0;
    guarded([&] { f = nb(net).getConvFlops(); });
    return f;
}

static void copyOut(const std::vector<float> &v, float *out, long long cap, long long *n_out)
{
    if (n_out) *n_out = static_cast<long long>(v.size());
    if (out && cap > 0) std::memcpy(out, v.data(), sizeof(float) * static_cast<size_t>(std::min<long long>(cap, static_cast<long long>(v.size()))));
}

int msnhnet_run_classify(msnhnet_t net, const float *img, long long n, float *out, long long cap, long long *n_out)
{
    return guarded([&] {
        if (!img || n <= 0) MSNH_THROW("bad argument");
        copyOut(nb(net).runClassify(std::vector<float>(img, img + n)), out, cap, n_out);
    });
}

int msnhnet_run_classify_gpu(msnhnet_t net, const float *img, long long n, float *out, long long cap, long long *n_out)
{
    return guarded([&] {
        if (!img || n <= 0) MSNH_THROW("bad argument");
        copyOut(nb(net).runClassifyGPU(img, static_cast<size_t>(n)), out, cap, n_out);
    });
}

int msnhnet_run_yolo_gpu(msnhnet_t net, const float *img, long long n, int *counts, float *boxes, long long cap_boxes, long long *total)
{
    return guarded([&] {
        if (!img || n <= 0) MSNH_THROW("bad argument");
        packBoxes(nb(net).runYoloGPU(img, static_cast<size_t>(n)), counts, boxes, cap_boxes, total);
    });
}

int msnhnet_last_nms_on_device(msnhnet_t net, int *on_device)
{
    return guarded([&] {
        if (!on_device) MSNH_THROW("bad argument");
        *on_device = nb(net).lastNmsOnDevice() ? 1 : 0;
    });
}

int msnhnet_fp16_headroom(msnhnet_t net, const float *img, long long n, float *headroom)
{
    return guarded([&] {
        if (!img || n <= 0 || !headroom) MSNH_THROW("bad argument");
        *headroom = nb(net).fp16Headroom(std::vector<float>(img, img + n));
    });
}

long long msnhnet_layer_output(msnhnet_t net, int layer, float *dst, long long cap)
{
    long long n = -1;
    guarded([&] {
        const std::vector<std::vector<float>> &outs = nb(net).layerOutputs();
        if (layer < 0 || static_cast<size_t>(layer) >= outs.size()) MSNH_THROW("no dump for this layer (enable msnhnet_set_save_layer_output and run)");
        const std::vector<float> &v = outs[static_cast<size_t>(layer)];
        n = static_cast<long long>(v.size());
        if (dst && cap > 0) std::memcpy(dst, v.data(), sizeof(float) * static_cast<size_t>(std::min(cap, n)));
    });
    return n;
}

long long msnhnet_yolo_head_logits(msnhnet_t net, int head, float *dst, long long cap)
{
    long long n = -1;
    guarded([&] {
        const std::vector<float> v = nb(net).yoloHeadLogits(head);
        n = static_cast<long long>(v.size());
        if (dst && cap > 0) std::memcpy(dst, v.data(), sizeof(float) * static_cast<size_t>(std::min(cap, n)));
    });
    return n;
}

long long msnhnet_yolo_candidates(msnhnet_t net, int image, float *dst, long long cap_rows)
{
    long long n = -1;
    guarded([&] {
        const std::vector<float> v = nb(net).yoloLastCandidates(image);
        n = static_cast<long long>(v.size() / 8);
        if (dst && cap_rows > 0) std::memcpy(dst, v.data(), sizeof(float) * 8 * static_cast<size_t>(std::min(cap_rows, n)));
    });
    return n;
}

int msnhnet_device_input(msnhnet_t net, float **device_ptr)
{
    return guarded([&] { if (!device_ptr) MSNH_THROW("pointer is NULL"); *device_ptr = nb(net).deviceInputBuffer(); });
}

int msnhnet_set_copy_on_forward_stream(msnhnet_t net, int on)
{
    return guarded([&] {
        Network *n = nb(net).getNet();
        if (n == nullptr || n->layers.empty() || n->layers.back()->type() != LayerType::YOLO_OUT) MSNH_THROW("not a yolo net");
        static_cast<YoloOutLayer *>(n->layers.back())->copyOnForwardStream = on != 0;
    });
}

int msnhnet_enqueue(msnhnet_t net, const float *device_input) { return guarded([&] { nb(net).enqueueForward(device_input); }); }
int msnhnet_sync(msnhnet_t net) { return guarded([&] { nb(net).sync(); }); }

int msnhnet_fetch_classify(msnhnet_t net, float *out, long long cap, long long *n_out)
{
    return guarded([&] { copyOut(nb(net).fetchClassify(), out, cap, n_out); });
}

int msnhnet_fetch_yolo(msnhnet_t net, int *counts, float *boxes, long long cap_boxes, long long *total)
{
    return guarded([&] { packBoxes(nb(net).fetchYolo(), counts, boxes, cap_boxes, total); });
}

int msnhnet_profile_ops(msnhnet_t net, int kind, int reps, float *ms_total, int *launches, double *flops)
{
    return guarded([&] {
        if (reps <= 0 || !ms_total) MSNH_THROW("bad argument");
        *ms_total = nb(net).profileOps(kind, reps, launches, flops);
    });
}

int msnhnet_profile_ops_bytes(msnhnet_t net, int kind, int reps, float *ms_total, int *launches, double *flops, double *bytes)
{
    return guarded([&] {
        if (reps <= 0 || !ms_total) MSNH_THROW("bad argument");
        *ms_total = nb(net).profileOps(kind, reps, launches, flops, bytes);
    });
}

long long msnhnet_profile_each_op_values(msnhnet_t net, int reps, double *dst, long long cap_rows)
{
    long long n = -1;
    guarded([&] {
        std::vector<double> v;
        nb(net).profileEachOp(reps > 0 ? reps : 1, &v);
        n = static_cast<long long>(v.size() / 8);
        if (dst && cap_rows > 0) std::memcpy(dst, v.data(), sizeof(double) * 8 * static_cast<size_t>(std::min(cap_rows, n)));
    });
    return n;
}

long long msnhnet_profile_each_op(msnhnet_t net, int reps, char *dst, long long cap)
{
    static thread_local std::string cache;
    long long n = -1;
    guarded([&] {
        if (dst == nullptr || cache.empty()) cache = nb(net).profileEachOp(reps > 0 ? reps : 1);
        n = copyText(cache, dst, cap);
        if (dst != nullptr) cache.clear();
    });
    return n;
}

long long msnhnet_yolo_max_boxes(msnhnet_t net)
{
    long long n = 0;
    guarded([&] {
        Network *nw = nb(net).getNet();
        long long cells = 0;
        for (const BaseLayer *l : nw->layers)
            if (l->type() == LayerType::YOLO) cells += 3LL * l->getOutHeight() * l->getOutWidth();
        n = cells * nw->batch;
    });
    return n;
}

int msnhnet_set_input_image_u8(msnhnet_t net, int index, const unsigned char *rgb_hwc, int width, int height, int half_init, int shuffle_rgb)
{
    return guarded([&] { nb(net).setInputImageU8(index, rgb_hwc, width, height, half_init != 0, shuffle_rgb != 0); });
}

int msnhnet_set_input_image(msnhnet_t net, int index, const unsigned char *rgb_hwc, int width, int height, int preproc, const float *mean3,
                            const float *std3, int shuffle_rgb)
{
    return guarded([&] { nb(net).setInputImage(index, rgb_hwc, width, height, preproc, mean3, std3, shuffle_rgb != 0); });
}

int msnhnet_boxes_to_image(float *boxes, long long count, int net_w, int net_h, int org_w, int org_h, int padded)
{
    return guarded([&] {
        if (count < 0 || (count > 0 && boxes == nullptr) || net_w <= 0 || net_h <= 0 || org_w <= 0 || org_h <= 0) MSNH_THROW("bad argument");
        for (long long i = 0; i < count; ++i)
        {
            float *r = boxes + 7 * i;
            YoloBox b;
            b.xywhBox = Box::XYWHBox(r[0], r[1], r[2], r[3]);
            if (padded) YoloOutLayer::bboxResize2Org(b, Point2I(net_w, net_h), Point2I(org_w, org_h));
            else        YoloOutLayer::bboxResize2OrgNoPad(b, Point2I(net_w, net_h), Point2I(org_w, org_h));
            r[0] = b.xywhBox.x; r[1] = b.xywhBox.y; r[2] = b.xywhBox.w; r[3] = b.xywhBox.h;
        }
    });
}

int msnhnet_boxes_from_candidates(const float *rows8, long long n, float nms_thresh, int fast, float *out, long long cap, long long *n_out)
{
    return guarded([&] {
        if ((!rows8 && n > 0) || n < 0 || n > (1LL << 30)) MSNH_THROW("bad argument");
        const std::vector<YoloBox> in = YoloOutLayer::sortedCandidates(rows8, static_cast<int>(n), nullptr, 0);
        std::vector<std::vector<YoloBox>> res(1);
        res[0] = fast ? YoloOutLayer::nmsSorted(in, nms_thresh) : YoloOutLayer::nms(in, nms_thresh, false);
        packBoxes(res, nullptr, out, cap, n_out);
    });
}

int msnhnet_nms(const float *rows, long long n, float nms_thresh, int fast, float *out, long long cap, long long *n_out)
{
    return guarded([&] {
        if ((!rows && n > 0) || n < 0) MSNH_THROW("bad argument");
        std::vector<YoloBox> in(static_cast<size_t>(n));
        for (long long i = 0; i < n; ++i)
        {
            const float *r = rows + 7 * i;
            YoloBox &b = in[static_cast<size_t>(i)];
            b.xywhBox = Box::XYWHBox(r[0], r[1], r[2], r[3]);
            b.conf = r[4]; b.bestClsConf = r[5]; b.bestClsIdx = static_cast<int>(r[6]);
        }
        std::vector<std::vector<YoloBox>> res(1);
        res[0] = fast ? YoloOutLayer::nmsSorted(in, nms_thresh) : YoloOutLayer::nms(in, nms_thresh, false);
        packBoxes(res, nullptr, out, cap, n_out);
    });
}

float msnhnet_gpu_inference_time(msnhnet_t net)
{
    float t = -1.f;
    guarded([&] { t = nb(net).getGpuInferenceTime(); });
    return t;
}

}

extern "C" {

static NetGroup &ng(msnhnet_group_t g)
{
    if (g == nullptr) MSNH_THROW("group handle is NULL");
    return *static_cast<NetGroup *>(g);
}

int msnhnet_group_create(const char *msnhnet_path, const char *msnhbin_path, int instances, int depth, msnhnet_group_t *group)
{
    return guarded([&] {
        if (!msnhnet_path || !msnhbin_path || !group) MSNH_THROW("NULL argument");
        *group = new NetGroup(msnhnet_path, msnhbin_path, instances, depth);
    });
}

int msnhnet_group_destroy(msnhnet_group_t group) { return guarded([&] { delete static_cast<NetGroup *>(group); }); }

int msnhnet_group_info(msnhnet_group_t group, int *instances, int *depth, int *is_detector)
{
    return guarded([&] {
        NetGroup &g = ng(group);
        if (instances) *instances = g.instances();
        if (depth) *depth = g.depth();
        if (is_detector) *is_detector = g.isDetector() ? 1 : 0;
    });
}

int msnhnet_group_instance(msnhnet_group_t group, int i, msnhnet_t *net)
{
    return guarded([&] {
        if (!net) MSNH_THROW("net pointer is NULL");
        if (i < 0 || i >= ng(group).instances()) MSNH_THROW("no such instance");
        *net = &ng(group).instance(i);
    });
}

int msnhnet_group_prime(msnhnet_group_t group, const float *device_input) { return guarded([&] { ng(group).prime(device_input); }); }
int msnhnet_group_submit(msnhnet_group_t group, const float *device_input) { return guarded([&] { ng(group).submit(device_input); }); }
int msnhnet_group_flush(msnhnet_group_t group) { return guarded([&] { ng(group).flush(); }); }

int msnhnet_group_fetch_classify(msnhnet_group_t group, float *out, long long cap, long long *n_out)
{
    return guarded([&] { copyOut(ng(group).fetchClassify(), out, cap, n_out); });
}

int msnhnet_group_fetch_yolo(msnhnet_group_t group, int *counts, float *boxes, long long cap_boxes, long long *total)
{
    return guarded([&] { packBoxes(ng(group).fetchYolo(), counts, boxes, cap_boxes, total); });
}

}
