// TEST INFRASTRUCTURE ONLY -- never linked into, imported by or shipped with the product.
//
// C-ABI shim over the *reference* CPU forward.  It is compiled by oracle/Makefile together with
// the reference's own sources where they lie under /root/reference (nothing is copied) into
// oracle/_ref/libmsnh_ref.so.  The shim only drives public reference entry points:
//   NetBuilder::buildNetFromMsnhNet   (src/net/MsnhNetBuilder.cpp:68-622)
//   NetBuilder::loadWeightsFromMsnhBin (src/net/MsnhNetBuilder.cpp:624-663)
//   the layer loop of runClassify/runYolo (src/net/MsnhNetBuilder.cpp:686-728, 763-806),
//   restated here only so that every layer's output can be captured the way the reference's own
//   setSaveLayerOutput dump does (src/net/MsnhNetBuilder.cpp:704-720);
//   the C facade runClassifyList / runYoloList (src/c_api/MsnhnetLib.cpp:540-905) through ref_facade_*.
#include <vector>
#include <string>
#include <cstring>
#include <cstdio>
#include <memory>
#include <exception>
#include <sstream>
#include <iostream>
#include <map>
#include <algorithm>
#include <chrono>
#include <cstdint>

#define private public      // NetBuilder::_netState has no getter; the capture loop needs the pools
#include "Msnhnet/net/MsnhNetBuilder.h"
#include "Msnhnet/utils/MsnhCVUtil.h"
#undef private

using namespace Msnhnet;

namespace {
struct RefNet
{
    NetBuilder                        *nb = nullptr;
    std::vector<std::vector<float>>    captured;     // per top-level layer output of the last run
    std::vector<std::vector<YoloBox>>  boxes;        // finalOut of the last run (yolo nets)
    std::string                        detail;
    double                             lastWallMs = 0;
};

void setErr(char *err, int errLen, const std::string &msg)
{
    if(err && errLen > 0)
    {
        std::snprintf(err, static_cast<size_t>(errLen), "%s", msg.c_str());
    }
}
}

extern "C" {

// scalarMode!=0: BaseLayer::supportAvx/supportFma=false, i.e. the scalar branches of the reference
// (the AVX max-pool branch is wrong for stride-1 padded pools, src/layers/MsnhMaxPoolLayer.cpp:517-544).
void *ref_create(int scalarMode)
{
    RefNet *r = new RefNet();
    std::streambuf *old = std::cout.rdbuf(nullptr);     // silence the SIMD banner (MsnhBaseLayer.cpp:21-59)
    r->nb = new NetBuilder();
    std::cout.rdbuf(old);
    if(scalarMode)
    {
        BaseLayer::supportAvx = false;
        BaseLayer::supportFma = false;
    }
    return r;
}

void ref_destroy(void *h)
{
    RefNet *r = static_cast<RefNet*>(h);
    if(!r) return;
    delete r->nb;
    delete r;
}

int ref_build(void *h, const char *msnhnetPath, char *err, int errLen)
{
    RefNet *r = static_cast<RefNet*>(h);
    try
    {
        r->nb->buildNetFromMsnhNet(msnhnetPath);
    }
    catch(const Exception &e)
    {
        setErr(err, errLen, e.what());
        return -1;
    }
    catch(const std::exception &e)
    {
        setErr(err, errLen, std::string("std: ") + e.what());
        return -2;
    }
    return 0;
}

int ref_load(void *h, const char *msnhbinPath, char *err, int errLen)
{
    RefNet *r = static_cast<RefNet*>(h);
    try
    {
        r->nb->loadWeightsFromMsnhBin(msnhbinPath);
    }
    catch(const Exception &e)
    {
        setErr(err, errLen, e.what());
        return -1;
    }
    catch(const std::exception &e)
    {
        setErr(err, errLen, std::string("std: ") + e.what());
        return -2;
    }
    return 0;
}

int ref_num_layers(void *h)
{
    RefNet *r = static_cast<RefNet*>(h);
    return static_cast<int>(r->nb->getNet()->layers.size());
}

// info[0..9] = type, outH, outW, outC, outputNum, inputNum, numWeights, memReUse, batch, activation
int ref_layer_info(void *h, int i, long long *info, char *name, int nameLen)
{
    RefNet *r = static_cast<RefNet*>(h);
    Network *net = r->nb->getNet();
    if(i < 0 || i >= static_cast<int>(net->layers.size())) return -1;
    BaseLayer *l = net->layers[static_cast<size_t>(i)];
    info[0] = static_cast<long long>(l->type());
    info[1] = l->getOutHeight();
    info[2] = l->getOutWidth();
    info[3] = l->getOutChannel();
    info[4] = l->getOutputNum();
    info[5] = l->getInputNum();
    info[6] = static_cast<long long>(l->getNumWeights());
    info[7] = l->getMemReUse();
    info[8] = l->getBatch();
    info[9] = static_cast<long long>(l->getActivation());
    setErr(name, nameLen, l->getLayerName());
    return 0;
}

long long ref_layer_detail(void *h, char *dst, long long cap)
{
    RefNet *r = static_cast<RefNet*>(h);
    r->detail = r->nb->getLayerDetail();
    long long n = static_cast<long long>(r->detail.size());
    if(dst && cap > 0)
    {
        long long c = std::min(n, cap - 1);
        std::memcpy(dst, r->detail.data(), static_cast<size_t>(c));
        dst[c] = 0;
    }
    return n;
}

// One batch-1 forward with the reference's own layer loop.  capture!=0 keeps every top-level layer's
// output.  Returns 0, or -1 with the reference's exception text.
int ref_run(void *h, const float *img, long long n, int capture, char *err, int errLen)
{
    RefNet *r = static_cast<RefNet*>(h);
    NetBuilder *nb = r->nb;
    Network *net = nb->getNet();
    NetworkState *st = nb->_netState;
    try
    {
        std::vector<float> in(img, img + n);
        r->captured.clear();
        r->boxes.clear();
        st->input    = in.data();
        st->inputNum = static_cast<int>(in.size());
        if(net->layers[0]->getInputNum() != st->inputNum)
        {
            throw Exception(1, "input image size err. Needed :" + std::to_string(net->layers[0]->getInputNum()) + " given :" +
                            std::to_string(in.size()), __FILE__, __LINE__, __FUNCTION__);
        }
        auto t0 = std::chrono::steady_clock::now();
        for(size_t i = 0; i < net->layers.size(); ++i)
        {
            BaseLayer *l = net->layers[i];
            l->forward(*st);
            if(l->getMemReUse() == 0)
            {
                st->input = l->getOutput();
            }
            st->inputNum = l->getOutputNum();
            if(capture)
            {
                const float *p = (l->getMemReUse() == 1) ? st->getInput() : st->input;
                r->captured.emplace_back(p, p + st->inputNum);
            }
        }
        auto t1 = std::chrono::steady_clock::now();
        r->lastWallMs = std::chrono::duration<double, std::milli>(t1 - t0).count();
        BaseLayer *last = net->layers.back();
        if(last->type() == LayerType::YOLO_OUT)
        {
            r->boxes = reinterpret_cast<YoloOutLayer*>(last)->finalOut;
        }
        if(!capture)
        {
            const float *p = (last->getMemReUse() == 1) ? st->getInput() : st->input;
            r->captured.assign(net->layers.size(), std::vector<float>());
            r->captured.back().assign(p, p + st->inputNum);
        }
    }
    catch(const Exception &e)
    {
        setErr(err, errLen, e.what());
        return -1;
    }
    catch(const std::exception &e)
    {
        setErr(err, errLen, std::string("std: ") + e.what());
        return -2;
    }
    return 0;
}

double ref_last_wall_ms(void *h)
{
    return static_cast<RefNet*>(h)->lastWallMs;
}

// The reference's own sum of per-layer forward times (src/net/MsnhNetBuilder.cpp:1159-1168), ms.
float ref_inference_time(void *h)
{
    return static_cast<RefNet*>(h)->nb->getInferenceTime();
}

long long ref_layer_output(void *h, int i, float *dst, long long cap)
{
    RefNet *r = static_cast<RefNet*>(h);
    if(i < 0 || i >= static_cast<int>(r->captured.size())) return -1;
    const std::vector<float> &v = r->captured[static_cast<size_t>(i)];
    long long n = static_cast<long long>(v.size());
    if(dst)
    {
        std::memcpy(dst, v.data(), sizeof(float) * static_cast<size_t>(std::min(n, cap)));
    }
    return n;
}

// Boxes of image 0 of the last run: rows of 7 floats  x y w h conf bestClsConf bestClsIdx.
long long ref_boxes(void *h, float *dst, long long capBoxes)
{
    RefNet *r = static_cast<RefNet*>(h);
    if(r->boxes.empty()) return 0;
    const std::vector<YoloBox> &b = r->boxes[0];
    long long n = static_cast<long long>(b.size());
    if(dst)
    {
        for(long long i = 0; i < std::min(n, capBoxes); ++i)
        {
            const YoloBox &q = b[static_cast<size_t>(i)];
            float *o = dst + 7 * i;
            o[0] = q.xywhBox.x; o[1] = q.xywhBox.y; o[2] = q.xywhBox.w; o[3] = q.xywhBox.h;
            o[4] = q.conf; o[5] = q.bestClsConf; o[6] = static_cast<float>(q.bestClsIdx);
        }
    }
    return n;
}

// CVUtil::getPaddingZeroF32C3 on a 3-channel 8-bit HWC image; dst holds 3*netW*netH floats (CHW).
int ref_letterbox_u8(const unsigned char *img, int width, int height, int netW, int netH, int halfInit, int shuffleRGB,
                     float *dst, char *err, int errCap)
{
    try
    {
        Mat mat(width, height, MAT_RGB_U8, const_cast<unsigned char*>(img));
        std::vector<float> v = CVUtil::getPaddingZeroF32C3(mat, Vec2I32(netW, netH), halfInit != 0 ? 1.f : 0.f, shuffleRGB != 0);
        std::memcpy(dst, v.data(), v.size() * sizeof(float));
        return 0;
    }
    catch(Exception &e)
    {
        std::snprintf(err, static_cast<size_t>(errCap), "%s", e.what());
        return 1;
    }
}

// The plain-resize pre-processing variants of CVUtil on a 3-channel 8-bit HWC image; dst holds 3*netW*netH floats (CHW).
// kind: 0 getImgDataF32C3, 1 the same with halfInit, 2 getGoogLenetF32C3, 3 getTransformedF32C3(mean, std), 4 getCaffeModeF32C3.
int ref_preproc_u8(const unsigned char *img, int width, int height, int netW, int netH, int kind, const float *mean, const float *stdv,
                   int shuffleRGB, float *dst, char *err, int errCap)
{
    try
    {
        Mat mat(width, height, MAT_RGB_U8, const_cast<unsigned char*>(img));
        std::vector<float> v;
        const Vec2I32 size(netW, netH);
        switch(kind)
        {
        case 0: v = CVUtil::getImgDataF32C3(mat, size, false, shuffleRGB != 0); break;
        case 1: v = CVUtil::getImgDataF32C3(mat, size, true, shuffleRGB != 0); break;
        case 2: v = CVUtil::getGoogLenetF32C3(mat, size, shuffleRGB != 0); break;
        case 3: v = CVUtil::getTransformedF32C3(mat, size, Vec3F32(mean[0], mean[1], mean[2]), Vec3F32(stdv[0], stdv[1], stdv[2]), shuffleRGB != 0); break;
        case 4: v = CVUtil::getCaffeModeF32C3(mat, size, shuffleRGB != 0); break;
        default: throw Exception(1, "unknown kind", __FILE__, __LINE__, __FUNCTION__);
        }
        std::memcpy(dst, v.data(), v.size() * sizeof(float));
        return 0;
    }
    catch(Exception &e)
    {
        std::snprintf(err, static_cast<size_t>(errCap), "%s", e.what());
        return 1;
    }
}

// YoloOutLayer::bboxResize2Org / bboxResize2OrgNoPad on one box given as x y w h; in place.
void ref_bbox_resize2org(float *xywh, int curW, int curH, int orgW, int orgH, int noPad)
{
    YoloBox b;
    b.xywhBox = Box::XYWHBox(xywh[0], xywh[1], xywh[2], xywh[3]);
    if(noPad) YoloOutLayer::bboxResize2OrgNoPad(b, Point2I(curW, curH), Point2I(orgW, orgH));
    else      YoloOutLayer::bboxResize2Org(b, Point2I(curW, curH), Point2I(orgW, orgH));
    xywh[0] = b.xywhBox.x; xywh[1] = b.xywhBox.y; xywh[2] = b.xywhBox.w; xywh[3] = b.xywhBox.h;
}

// ---- the reference's own C facade (src/c_api/MsnhnetLib.cpp, the build without OpenCV: :463-905), compiled from its source by
// oracle/Makefile.  Its functions are declared here by hand: its header pulls in the umbrella header of the whole project.
// The facade keeps one process-wide network (MsnhnetLib.cpp:3); the wrappers below drive it on the CPU (runGPU = 0).
struct RefFacadeBBox { float x, y, w, h, conf, bestClsConf; uint32_t bestClsIdx; float angle; };      // MsnhnetLib.h:22-32
struct RefFacadeBBoxContainer { RefFacadeBBox boxes[1024]; };                                            // MsnhnetLib.h:9, :34-37
int initMsnhnet();
int buildMsnhnet(char **msg, const char *msnhnet, const char *msnhbin, int useFp16, int useCudaOnly);
int runClassifyList(char **msg, unsigned char *imageData, const int width, const int height, const int channel, int *bestIndex,
                    int preDataType, const int swapRGB, int runGPU, const float *mean, const float *std);
int runYoloList(char **msg, unsigned char *imageData, const int width, const int height, const int channel,
                RefFacadeBBoxContainer *bboxContainer, int *detectedNum, const int swapRGB, const int runGPU);
int dispose();

// initMsnhnet + buildMsnhnet; scalarMode as for ref_create.  Returns the facade's own code (1 = success).
int ref_facade_build(const char *msnhnetPath, const char *msnhbinPath, int scalarMode)
{
    std::streambuf *old = std::cout.rdbuf(nullptr);
    initMsnhnet();
    std::cout.rdbuf(old);
    if(scalarMode)
    {
        BaseLayer::supportAvx = false;
        BaseLayer::supportFma = false;
    }
    char *msg = nullptr;                // on failure the facade leaves a pointer into a destroyed vector here (:29-31): never read
    return buildMsnhnet(&msg, msnhnetPath, msnhbinPath, 0, 0);
}

// runClassifyList on a private copy of a 3-channel image (the facade converts its argument in place, :562-565)
int ref_facade_classify_list(const unsigned char *img, int width, int height, int preDataType, int swapRGB, const float *mean,
                             const float *stdv, int *bestIndex)
{
    std::vector<unsigned char> copy(img, img + static_cast<size_t>(width) * height * 3);
    char *msg = nullptr;
    return runClassifyList(&msg, copy.data(), width, height, 3, bestIndex, preDataType, swapRGB, 0, mean, stdv);
}

// runYoloList likewise; dst receives rows of 7 floats (x y w h conf bestClsConf bestClsIdx), *count the number of boxes
int ref_facade_yolo_list(const unsigned char *img, int width, int height, int swapRGB, float *dst, int capBoxes, int *count)
{
    std::vector<unsigned char> copy(img, img + static_cast<size_t>(width) * height * 3);
    std::unique_ptr<RefFacadeBBoxContainer> box(new RefFacadeBBoxContainer());
    char *msg = nullptr;
    *count = 0;
    const int rc = runYoloList(&msg, copy.data(), width, height, 3, box.get(), count, swapRGB, 0);
    if(rc != 1) return rc;
    for(int i = 0; i < *count && i < capBoxes; ++i)
    {
        const RefFacadeBBox &q = box->boxes[i];
        float *o = dst + 7 * i;
        o[0] = q.x; o[1] = q.y; o[2] = q.w; o[3] = q.h; o[4] = q.conf; o[5] = q.bestClsConf; o[6] = static_cast<float>(q.bestClsIdx);
    }
    return rc;
}

int ref_facade_dispose() { return dispose(); }

void ref_set_threads_note(int *ompMax)
{
#ifdef USE_OMP
    *ompMax = OMP_THREAD;
#else
    *ompMax = 1;
#endif
}

}
