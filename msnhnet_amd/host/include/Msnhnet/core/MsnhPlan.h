// The device plan of one network: the flat list of kernel launches ("ops") a graph lowers to, the tensors
// they read and write, and the single device arena those tensors are placed in.
//
// The reference allocates per layer: two ping-pong pools sized for the largest output plus an own buffer
// for every layer that is re-read later (src/net/MsnhNetBuilder.cpp:539-589), and its block layers
// malloc/free a copy of their input on every forward (src/layers/MsnhResBlockLayer.cpp:319,391).  Here the
// whole graph -- block internals included -- is lowered once, then
//   1. fused   : conv + stand-alone batch-norm, conv + residual add (+ block activation) become one launch;
//   2. aliased : route / concat-block inputs are placed directly inside the concatenated tensor (a channel
//                slice with a larger pixel stride), so the concat copy disappears;
//   3. scaled  : for float16, one float32 calibration pass fixes a power-of-two scale per tensor so that
//                activations far outside the half range still fit (the scale is applied exactly in the
//                float32 epilogues);
//   4. placed  : tensor lifetimes over the op list drive a first-fit assignment of arena offsets.
#pragma once
#include <array>
#include <memory>
#include <string>
#include <vector>
#include "Msnhnet/config/MsnhnetCfg.h"
#include "Msnhnet/core/MsnhDevice.h"
#include "Msnhnet/core/MsnhPackFile.h"

namespace Msnhnet
{
class BaseLayer;

struct PlanTensor
{
    enum Layout { NHWC = 0, NCHW_INPUT, FLAT };
    int  n = 0, h = 0, w = 0, c = 0;
    int  dtype = MSNH_F32;
    Layout layout = NHWC;
    int  parent = -1;          // >= 0: this tensor is channels [chanOffset, chanOffset+c) of `parent`
    int  chanOffset = 0;
    int  scaleExp = 0;         // stored value = true value * 2^-scaleExp
    bool pinned = false;       // must stay a real tensor (top-level outputs while layer dumps are on, ...)
    bool persistent = false;   // must survive until the end of the forward
    int  ld = 0;               // pixel stride in elements (root tensors)
    size_t bytes = 0;          // root tensors
    size_t offset = 0;         // arena offset (root tensors)
    bool external = false;     // storage provided outside the arena (the network input)
    void *extPtr = nullptr;
    float amax = 0.f;          // calibration result
    std::string name;
    size_t elems() const { return static_cast<size_t>(n) * h * w * c; }
    long long pixels() const { return static_cast<long long>(n) * h * w; }
};

struct PlanOp
{
    enum Kind { CONV = 0, AFFINE, ADD, COPY, MAXPOOL, AVGPOOL, UPSAMPLE, CONNECTED, INPUT_CAST, YOLO_DECODE, PAD, SLICE, BILINEAR, SOFTMAX, COL2IM };
    Kind kind = CONV;
    int  in0 = -1, in1 = -1, out = -1;
    bool dead = false;
    int  layerIndex = -1;      // top-level layer this op belongs to
    std::string name;

    // geometry / epilogue
    int  ksize = 1, stride = 1, pad = 0, dilation = 1, groups = 1;
    ActivationType act = NONE, act2 = NONE;
    float actParam = 0.1f, act2Param = 0.1f;
    float upScale = 1.f;                    // UPSAMPLE: value scale; SOFTMAX: temperature
    int  dstChanOffset = 0;                 // COPY: channel offset inside `out`
    bool pureAct = false;                   // AFFINE with identity scale and shift: only the activation matters
    float in1Sign = 1.f;                    // ADD: out = act(in0 + in1Sign * in1); CONV with a fused add: sign of the residual
    int  padTop = 0, padLeft = 0;           // PAD
    float padValue = 0.f;
    int  slice[6] = {0, 1, 0, 1, 0, 1};     // SLICE: start / step of channels, rows, columns
    int  alignCorners = 0;                  // BILINEAR
    int  yoloVersion = 3;                   // YOLO_DECODE: 3, 4 or 5
    int  algo = MSNH_CONV_AUTO;             // CONV: resolved at weight preparation
    int  tile = 0;                          // CONV/IGEMM: tile configuration chosen by Plan::tuneConvs (0 = library default)
    BaseLayer *src = nullptr;               // layer that owns the host weights of this op
    BaseLayer *src2 = nullptr;              // batch-norm layer folded into a CONV
    int  chainHead = -1;                    // MAXPOOL: >= 0 = this pool's result is written by the launch of op chainHead (a chain of stride-1 pools in one launch)
    int  chainNext = -1;                    // MAXPOOL at the head or inside such a chain: the op whose pool follows
    int  stemOp = -1;                       // CONV 3x3 stride 2: the (dead) first-layer op computed in front of it by the same launch (Plan::fuse c)
    bool up2 = false;                       // CONV: the launch writes every result pixel to the 2 x 2 pixels of `out` it maps to (Plan::fuse f): `out` is the
                                            // tensor of the (dead) nearest-neighbour upsample that read this convolution's result
    int  stemTail = -1;                     // CONV with stemOp: the (dead) 1x1 convolution with 32 filters that reads this op's result, computed by the
                                            // same launch (Plan::fuse c, msnh_hip_conv_stem_down_tail)
    int  mbExpand = -1, mbDw = -1;          // CONV 1x1 closing an inverted-residual block: the (dead) 1x1 expand and 3x3 depthwise ops computed in front of
                                            // it by the same launch (Plan::fuse d, msnh_hip_mbconv)

    int  tail = -1;                         // CONV: the 1x1 convolution op that reads this one's result and that the same launch can compute
                                            // (Plan::fuse e); it does when the search set algo to MSNH_CONV_IGEMM_TAIL, and the 1x1 op is then dead
    int  tailOf = -1;                       // CONV 1x1: the op whose launch may compute it
    double ownFlops = 0;                    // CONV with a tail: flops without the tail's
    bool tailSkipY = false;                 // CONV computing its tail: nothing but the tail reads this op's own result, which therefore is not written

    // YOLO_DECODE
    std::array<float, 6> anchors{};
    int   classes = 0;
    float ratio = 1.f;
    int   cellBase = 0;                     // first cell of this head inside an image's decoded rows
    float confThresh = 0.f;

    // device-side constants, filled by Plan::prepareWeights
    DeviceBuffer wDev, scaleDev, shiftDev;
    DeviceBuffer wDev2, scaleDev2, shiftDev2;   // stemOp >= 0: the first layer's
    DeviceBuffer wDev3, scaleDev3, shiftDev3;   // stemTail >= 0: the 1x1 convolution's
    double flops = 0;                       // 2*MACs of this launch (conv / connected)
};

class Plan
{
public:
    explicit Plan(int dtype) : computeDtype(dtype) {}

    int computeDtype;
    bool sparseYolo = false;                // yolo heads decode only the rows of their candidates (nobody reads the full decoded tensors)
    bool yoloKeepDecoded = true;            // sparseYolo: also write the candidates' full decoded rows (only YoloBox::classesVal needs them)
    std::vector<size_t> yoloHeadOps;        // sparseYolo: the heads' decode ops in cell order when one launch (issued at the last of them in
                                            // op order) can decode them all; empty = one launch pair per head
    void findYoloHeads();                   // fills yoloHeadOps; call once the heads' cell numbers are assigned
    bool fuseMbconv = true;                 // float16: 1x1 expand -> 3x3 depthwise -> 1x1 project as one launch where msnh_hip_mbconv takes the block
    bool fuseTail = false;                  // float16: a convolution whose tile holds all its output channels also computes the 1x1 convolution that
                                            // reads its result (msnh_hip_conv2d_tail), where the per-layer search finds that faster than two launches
    bool forceTail = false;                 // ... wherever the library takes the pair, whatever the timing says (tests)
    bool fuseUpsample = true;               // a convolution whose only reader is a 2x nearest-neighbour upsample writes the upsampled tensor itself
    bool fuseStemTail = true;               // ... and the 1x1 convolution with 32 filters behind that pair in the same launch (msnh_hip_conv_stem_down_tail)
    bool fuseStemDown = true;               // float16: first layer + first stride-2 layer as one launch where msnh_hip_conv_stem_down takes the pair
    bool preferWinograd = false;            // 3x3 stride-1 float16 convs take the Winograd path where the kernel accepts the shape
    std::vector<PlanTensor> tensors;
    std::vector<PlanOp>     ops;
    std::vector<int>        layerOut;       // output tensor of each top-level layer
    int inputTensor = -1;
    int inputNhwc = -1;                     // NHWC copy of the network input, made on first use by a non-convolution first layer

    // YOLO post-processing buffers (only for networks ending in a yoloout layer)
    int  yoloCells = 0;                     // sum over heads of 3*H*W
    int  yoloClasses = 0;
    DeviceBuffer yoloDecoded, yoloCandIdx, yoloCandCnt, yoloRows;

    int addTensor(int n, int h, int w, int c, int dtype, const std::string &name, PlanTensor::Layout layout = PlanTensor::NHWC);
    PlanOp &addOp(PlanOp::Kind kind, int in0, int in1, int out, int layerIndex, const std::string &name);
    int producerOf(int tensor) const;       // last live op writing `tensor`, or -1
    int nhwcOf(int tensor, int layerIndex); // `tensor` itself, or (for the NCHW network input) its NHWC copy in the compute dtype
    int consumerCount(int tensor) const;

    void fuse();                            // passes 1
    void chainMaxPools();                   // stride-1 max-pools of one tensor (SPP): each larger window reads the next smaller one's result
    void aliasConcats();                    // pass 2
    void applyCalibration(const std::vector<float> &amax);   // pass 3: amax per tensor, from an executed float32 twin (or from its record on disk)
    std::vector<float> amaxOfTensors() const;
    uint64_t structureHash() const;         // over ops and tensors as lowered and optimised (before placement): what a pack file must match
    void place();                           // pass 4 + arena allocation
    // fold batch-norm, pick algorithms, pack and upload weights; packed kernels are taken from `from` where it holds them and recorded in `to`
    void prepareWeights(PackFile *from = nullptr, PackFile *to = nullptr);
    // time every tile configuration / algorithm variant per conv launch, keep the fastest.  cacheFile (may be empty): choices of an
    // earlier search for the same plan on the same device are read from it instead of being timed again, and written to it otherwise
    void tuneConvs(msnh_stream_t s, const std::string &cacheFile = std::string());
    void run(size_t opBegin, size_t opEnd, msnh_stream_t s);
    void runAll(msnh_stream_t s) { run(0, ops.size(), s); }
    float fp16Headroom(msnh_stream_t s);    // eager run on the current input: 65504 / largest stored float16 magnitude, 0 after an overflow
    void runCalibration(msnh_stream_t s);   // one eager run; absmax of every NHWC tensor taken right behind the launch that writes it

    int   root(int t) const;
    int   chanOffsetInRoot(int t) const;
    void *ptr(int t) const;
    int   ld(int t) const { return tensors[static_cast<size_t>(root(t))].ld; }
    float mulOf(int t) const;               // 2^scaleExp
    // Copies tensor `t` to the host as batch-major NCHW float32 true values.
    void  exportTensor(int t, std::vector<float> &dst, msnh_stream_t s);

    size_t arenaBytes() const { return _arena.bytes(); }
    size_t liveOps() const;                 // launches of one forward
    double totalConvFlops() const;
    std::string describe() const;           // one line per live op: kind, shapes, algorithm

private:
    void launch(PlanOp &op, msnh_stream_t s);
    void applyTails();                      // after the search: the 1x1 ops computed by their producer's launch become dead, the others alive
    DeviceBuffer _arena, _exportScratch, _convWorkspace;
    bool _tailWriteAll = false;             // runs that look at every tensor (calibration, float16 headroom): tailSkipY is ignored
};
}
