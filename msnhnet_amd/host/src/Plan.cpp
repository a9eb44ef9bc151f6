// Device plan: fusion, concat aliasing, float16 scale calibration, arena placement, weight preparation and
// the launch of every op through the kernel library's C ABI.
#include "Msnhnet/core/MsnhPlan.h"
#include <algorithm>
#include <cmath>
#include <cstring>
#include <cstdio>
#include <fstream>
#include <functional>
#include <limits>
#include <map>
#include <mutex>
#include <numeric>
#include <sstream>
#include "Msnhnet/layers/MsnhBaseLayer.h"

namespace Msnhnet
{
// ---- Device ---------------------------------------------------------------------------------------------
static bool g_deviceReady = false;
static std::mutex g_deviceMutex;

void Device::ensureInit()
{
    std::lock_guard<std::mutex> lock(g_deviceMutex);
    if (g_deviceReady) return;
    int count = 0;
    msnh_hip_device_count(&count);
    if (count <= 0) MSNH_THROW("no MI355X/HIP device is visible: this build has no CPU path");
    MSNH_DEV(msnh_hip_init(0));
    g_deviceReady = true;
}

bool Device::initialised() { return g_deviceReady; }

// ---- construction -------------------------------------------------------------------------------------------
int Plan::addTensor(int n, int h, int w, int c, int dtype, const std::string &name, PlanTensor::Layout layout)
{
    PlanTensor t;
    t.n = n; t.h = h; t.w = w; t.c = c; t.dtype = dtype; t.name = name; t.layout = layout;
    tensors.push_back(t);
    return static_cast<int>(tensors.size()) - 1;
}

PlanOp &Plan::addOp(PlanOp::Kind kind, int in0, int in1, int out, int layerIndex, const std::string &name)
{
    ops.emplace_back();
    PlanOp &op = ops.back();
    op.kind = kind; op.in0 = in0; op.in1 = in1; op.out = out; op.layerIndex = layerIndex; op.name = name;
    return op;
}

int Plan::nhwcOf(int tensor, int layerIndex)
{
    const PlanTensor t = tensors[static_cast<size_t>(tensor)];
    if (t.layout != PlanTensor::NCHW_INPUT) return tensor;
    if (inputNhwc < 0)
    {
        inputNhwc = addTensor(t.n, t.h, t.w, t.c, computeDtype, "input_nhwc");
        addOp(PlanOp::INPUT_CAST, tensor, -1, inputNhwc, layerIndex, "input_cast");
    }
    return inputNhwc;
}

int Plan::producerOf(int tensor) const
{
    for (int i = static_cast<int>(ops.size()) - 1; i >= 0; --i)
        if (!ops[static_cast<size_t>(i)].dead && ops[static_cast<size_t>(i)].out == tensor) return i;
    return -1;
}

int Plan::consumerCount(int tensor) const
{
    int n = 0;
    for (const PlanOp &op : ops)
        if (!op.dead) n += (op.in0 == tensor) + (op.in1 == tensor);
    return n;
}

size_t Plan::liveOps() const
{
    size_t n = 0;
    for (const PlanOp &op : ops) n += (op.dead || op.chainHead >= 0) ? 0 : 1;
    return n;
}

double Plan::totalConvFlops() const
{
    double f = 0;
    for (const PlanOp &op : ops)
        if (!op.dead) f += op.flops;
    return f;
}

int Plan::root(int t) const
{
    while (tensors[static_cast<size_t>(t)].parent >= 0) t = tensors[static_cast<size_t>(t)].parent;
    return t;
}

int Plan::chanOffsetInRoot(int t) const
{
    int off = 0;
    while (tensors[static_cast<size_t>(t)].parent >= 0)
    {
        off += tensors[static_cast<size_t>(t)].chanOffset;
        t = tensors[static_cast<size_t>(t)].parent;
    }
    return off;
}

void *Plan::ptr(int t) const
{
    const PlanTensor &r = tensors[static_cast<size_t>(root(t))];
    unsigned char *base = r.external ? static_cast<unsigned char *>(r.extPtr) : _arena.as<unsigned char>() + r.offset;
    if (base == nullptr) MSNH_THROW("plan tensor '" + tensors[static_cast<size_t>(t)].name + "' has no storage");
    const size_t el = r.dtype == MSNH_F16 ? 2 : 4;
    return base + static_cast<size_t>(chanOffsetInRoot(t)) * el;
}

float Plan::mulOf(int t) const { return std::ldexp(1.f, tensors[static_cast<size_t>(t)].scaleExp); }

// ---- pass 1: fusion ---------------------------------------------------------------------------------------------
void Plan::fuse()
{
    // (a) CONV (no activation) -> AFFINE on the conv's only consumer : fold the affine into the conv epilogue.
    for (size_t i = 0; i < ops.size(); ++i)
    {
        PlanOp &aff = ops[i];
        if (aff.dead || aff.kind != PlanOp::AFFINE) continue;
        const int p = producerOf(aff.in0);
        if (p < 0) continue;
        if (aff.pureAct)
        {
            // a stand-alone activation moves into whatever produced its input, if that has no activation of its own yet
            PlanOp &prod = ops[static_cast<size_t>(p)];
            if (tensors[static_cast<size_t>(aff.in0)].pinned || consumerCount(aff.in0) != 1) continue;
            if (prod.kind == PlanOp::CONV && prod.in1 >= 0)
            {
                if (prod.act2 != NONE) continue;
                prod.act2 = aff.act; prod.act2Param = aff.actParam;
            }
            else if (prod.kind == PlanOp::CONV || prod.kind == PlanOp::AFFINE || prod.kind == PlanOp::ADD || prod.kind == PlanOp::CONNECTED)
            {
                if (prod.act != NONE) continue;
                prod.act = aff.act; prod.actParam = aff.actParam;
            }
            else continue;
            prod.out = aff.out;
            aff.dead = true;
            continue;
        }
        PlanOp &conv = ops[static_cast<size_t>(p)];
        if (conv.kind != PlanOp::CONV || conv.act != NONE || conv.src2 != nullptr || conv.in1 >= 0) continue;
        if (tensors[static_cast<size_t>(aff.in0)].pinned || consumerCount(aff.in0) != 1) continue;
        conv.src2 = aff.src;
        conv.act = aff.act;
        conv.actParam = aff.actParam;
        conv.out = aff.out;
        aff.dead = true;
    }
    // (b) CONV -> ADD(conv output, other) : the add and the block activation move into the conv epilogue.
    for (size_t i = 0; i < ops.size(); ++i)
    {
        PlanOp &add = ops[i];
        if (add.dead || add.kind != PlanOp::ADD) continue;
        for (int side = 0; side < 2; ++side)
        {
            const int mine = side == 0 ? add.in0 : add.in1;
            const int other = side == 0 ? add.in1 : add.in0;
            const int p = producerOf(mine);
            if (p < 0 || mine == other) continue;
            PlanOp &conv = ops[static_cast<size_t>(p)];
            if (conv.kind != PlanOp::CONV || conv.in1 >= 0) continue;
            if (tensors[static_cast<size_t>(mine)].pinned || consumerCount(mine) != 1) continue;
            // a subtraction (in0 - in1) only moves into the epilogue of the conv that produces in0: the sign then rides
            // on the residual multiplier; -conv + other has no epilogue form
            if (side == 1 && add.in1Sign != 1.f) continue;
            // the other operand must already exist when the conv runs
            const int po = producerOf(other);
            if (po >= p) continue;
            conv.in1 = other;
            conv.in1Sign = side == 0 ? add.in1Sign : 1.f;
            conv.act2 = add.act;
            conv.act2Param = add.actParam;
            conv.out = add.out;
            add.dead = true;
            break;
        }
    }
    // (c) float16: first layer (3x3 stride 1, 32 filters, over the NCHW network input) -> 3x3 stride-2 convolution that is its only
    // consumer: one launch; the full-resolution 32-channel tensor between them stays on the chip (it keeps its place in the tensor
    // list: its calibrated scale is the scale of the values in LDS)
    if (computeDtype == MSNH_F16 && fuseStemDown)
        for (size_t i = 0; i < ops.size(); ++i)
        {
            PlanOp &first = ops[i];
            if (first.dead || first.kind != PlanOp::CONV || first.in1 >= 0 || first.groups != 1 || first.dilation != 1) continue;
            const PlanTensor &in = tensors[static_cast<size_t>(first.in0)];
            const PlanTensor &mid = tensors[static_cast<size_t>(first.out)];
            if (in.layout != PlanTensor::NCHW_INPUT || mid.pinned || mid.persistent || mid.parent >= 0 || mid.dtype != MSNH_F16 || consumerCount(first.out) != 1) continue;
            for (size_t k = i + 1; k < ops.size(); ++k)
            {
                PlanOp &down = ops[k];
                if (down.dead || down.in0 != first.out) continue;
                const PlanTensor &out = tensors[static_cast<size_t>(down.out)];
                if (down.kind == PlanOp::CONV && down.in1 < 0 && down.groups == 1 && down.dilation == 1 && out.dtype == MSNH_F16 && out.layout == PlanTensor::NHWC &&
                    msnh_hip_conv_stem_down_supported(in.c, mid.c, first.ksize, first.stride, first.pad, out.c, down.ksize, down.stride, down.pad))
                {
                    down.stemOp = static_cast<int>(i);
                    down.in0 = first.in0;
                    first.dead = true;
                    // ... and the 1x1 convolution with 32 filters that reads the pair's result (the opening of Darknet-53's first residual
                    // block), if it is the next launch: computed by the pair's launch from its own registers.  The pair's result is still
                    // written (the block's residual add reads it).
                    for (size_t t = k + 1; fuseStemTail && t < ops.size(); ++t)
                    {
                        PlanOp &tail = ops[t];
                        if (tail.dead) continue;
                        const PlanTensor &z = tensors[static_cast<size_t>(tail.out)];
                        if (tail.kind == PlanOp::CONV && tail.in0 == down.out && tail.in1 < 0 && tail.groups == 1 && tail.dilation == 1 && tail.stemOp < 0 &&
                            tail.mbExpand < 0 && z.dtype == MSNH_F16 && z.layout == PlanTensor::NHWC &&
                            msnh_hip_conv_stem_down_tail_supported(out.c, z.c, tail.ksize, tail.stride, tail.pad))
                        {
                            down.stemTail = static_cast<int>(t);
                            tail.dead = true;
                        }
                        break;
                    }
                }
                break;
            }
        }
    // (d) float16: 1x1 convolution -> 3x3 depthwise convolution -> 1x1 convolution, each the only consumer of the one before (the
    // inverted-residual block of MobileNetV2; the closing convolution may already carry the block's residual add from (b)): one launch,
    // the two widened tensors stay on the chip.  They keep their places in the tensor list: their calibrated scales are the scales of
    // the values in LDS.
    if (computeDtype == MSNH_F16 && fuseMbconv)
        for (size_t i = 0; i < ops.size(); ++i)
        {
            PlanOp &proj = ops[i];
            if (proj.dead || proj.kind != PlanOp::CONV || proj.ksize != 1 || proj.stride != 1 || proj.pad != 0 || proj.groups != 1 || proj.stemOp >= 0) continue;
            const auto inner = [&](int t) {
                const PlanTensor &pt = tensors[static_cast<size_t>(t)];
                return !pt.pinned && !pt.persistent && !pt.external && pt.parent < 0 && pt.dtype == MSNH_F16 && pt.layout == PlanTensor::NHWC && consumerCount(t) == 1;
            };
            const int pd = producerOf(proj.in0);
            if (pd < 0 || !inner(proj.in0)) continue;
            PlanOp &dw = ops[static_cast<size_t>(pd)];
            const PlanTensor &wide = tensors[static_cast<size_t>(dw.in0)];
            if (dw.kind != PlanOp::CONV || dw.ksize != 3 || dw.pad != 1 || dw.dilation != 1 || (dw.stride != 1 && dw.stride != 2) || dw.in1 >= 0 || dw.stemOp >= 0 ||
                dw.groups != wide.c || tensors[static_cast<size_t>(dw.out)].c != wide.c)
                continue;
            const int pe = producerOf(dw.in0);
            if (pe < 0 || !inner(dw.in0)) continue;
            PlanOp &ex = ops[static_cast<size_t>(pe)];
            if (ex.kind != PlanOp::CONV || ex.ksize != 1 || ex.stride != 1 || ex.pad != 0 || ex.groups != 1 || ex.in1 >= 0 || ex.stemOp >= 0 || ex.mbExpand >= 0) continue;
            const PlanTensor &in = tensors[static_cast<size_t>(ex.in0)];
            const PlanTensor &out = tensors[static_cast<size_t>(proj.out)];
            if (in.layout != PlanTensor::NHWC || in.dtype != MSNH_F16 || out.dtype != MSNH_F16 || out.layout != PlanTensor::NHWC) continue;
            // the residual must exist when the fused launch runs, which is where the closing convolution stands: it does
            msnh_mbconv_desc d;
            std::memset(&d, 0, sizeof(d));
            const auto up8 = [](int c) { return (c + 7) / 8 * 8; };
            d.batch = in.n; d.in_h = in.h; d.in_w = in.w; d.in_c = in.c; d.in_ld = up8(in.c);
            d.exp_c = wide.c; d.stride = dw.stride;
            d.out_c = out.c; d.out_h = out.h; d.out_w = out.w; d.out_ld = up8(out.c);
            d.act1 = static_cast<int>(ex.act); d.act2 = static_cast<int>(dw.act); d.act3 = static_cast<int>(proj.act); d.act4 = static_cast<int>(proj.act2);
            d.has_residual = proj.in1 >= 0 ? 1 : 0; d.res_ld = up8(out.c);
            d.mul1 = d.mul2 = d.out_mul = d.res_mul = 1.f;
            if (!msnh_hip_mbconv_supported(&d)) continue;
            proj.mbExpand = pe;
            proj.mbDw = pd;
            proj.in0 = ex.in0;
            ex.dead = true;
            dw.dead = true;
        }
    // (f) convolution -> 2x nearest-neighbour upsample that is its only reader (the lateral branches of the detection necks,
    // src/layers/MsnhUpSampleLayer.cpp:96-118 behind a 1x1 ConvolutionalLayer): the convolution's epilogue writes every result pixel to the
    // four pixels it maps to (msnh_conv_desc::out_upsample), the 19x19 / 38x38 tensor in between is never stored and the upsample launch goes.
    if (fuseUpsample)
        for (size_t i = 0; i < ops.size(); ++i)
        {
            PlanOp &up = ops[i];
            if (up.dead || up.kind != PlanOp::UPSAMPLE || up.stride != 2 || up.upScale != 1.f) continue;
            const int pc = producerOf(up.in0);
            if (pc < 0) continue;
            PlanOp &conv = ops[static_cast<size_t>(pc)];
            const PlanTensor &x = tensors[static_cast<size_t>(conv.in0)];
            const PlanTensor &mid = tensors[static_cast<size_t>(up.in0)];
            const PlanTensor &big = tensors[static_cast<size_t>(up.out)];
            const int vec = x.dtype == MSNH_F16 ? 8 : 4;
            if (conv.kind != PlanOp::CONV || conv.in1 >= 0 || conv.groups != 1 || conv.stemOp >= 0 || conv.mbExpand >= 0 || conv.up2 || conv.tail >= 0 ||
                conv.tailOf >= 0 || x.layout != PlanTensor::NHWC || x.c % vec != 0 || x.c <= 4 || mid.c % 8 != 0 || mid.pinned || mid.persistent || mid.external ||
                mid.parent >= 0 || consumerCount(up.in0) != 1 || mid.dtype != big.dtype || big.h != 2 * mid.h || big.w != 2 * mid.w ||
                (x.dtype == MSNH_F32 && mid.dtype != MSNH_F32))
                continue;
            conv.out = up.out;
            conv.up2 = true;
            up.dead = true;
        }
    // (e) float16: convolution -> 1x1 stride-1 convolution (the 3x3 that closes a Darknet residual block and the 1x1 that opens the next one,
    // src/layers/MsnhResBlockLayer.cpp:215-302): where one tile of the first launch holds all its output channels (at most 256) and the 1x1 has at
    // most 128 filters, the first launch can compute the 1x1 from its own result tile (msnh_hip_conv2d_tail).  Only marked here: both ops stay
    // alive, the per-layer search times the pair both ways (tuneConvs), and the 1x1's result is placed from the first launch on.
    if (computeDtype == MSNH_F16 && fuseTail)
        for (size_t i = 0; i < ops.size(); ++i)
        {
            PlanOp &b = ops[i];
            if (b.dead || b.kind != PlanOp::CONV || b.ksize != 1 || b.stride != 1 || b.pad != 0 || b.groups != 1 || b.in1 >= 0 || b.stemOp >= 0 || b.mbExpand >= 0 ||
                b.tail >= 0 || b.tailOf >= 0 || b.up2)
                continue;
            const int pa = producerOf(b.in0);
            if (pa < 0 || pa >= static_cast<int>(i)) continue;
            PlanOp &a = ops[static_cast<size_t>(pa)];
            if (a.kind != PlanOp::CONV || a.groups != 1 || a.dilation != 1 || a.stemOp >= 0 || a.mbExpand >= 0 || a.tail >= 0 || a.tailOf >= 0 || a.up2 || a.out != b.in0) continue;
            const PlanTensor &x = tensors[static_cast<size_t>(a.in0)];
            const PlanTensor &y = tensors[static_cast<size_t>(a.out)];
            const PlanTensor &z = tensors[static_cast<size_t>(b.out)];
            const auto f16Image = [](const PlanTensor &t) { return t.dtype == MSNH_F16 && t.layout == PlanTensor::NHWC; };
            if (!f16Image(x) || !f16Image(y) || !f16Image(z) || x.c % 8 != 0 || y.c % 8 != 0 || y.c > 256 || z.c % 8 != 0 || z.c > 128) continue;
            if (a.in1 >= 0 && !f16Image(tensors[static_cast<size_t>(a.in1)])) continue;
            a.tail = static_cast<int>(i);
            b.tailOf = pa;
        }
}

// ---- pass 1b: stride-1 max-pools over one tensor (SPP blocks: 5, 9, 13) ---------------------------------------------
// With -FLT_MAX padding and stride 1, a window of a + b - 1 is the window b over the result of the window a, exactly
// (max is associative and the clipped windows compose).  So the pools of one input run smallest first and each larger one
// reads its predecessor through the difference window: 5, 5 over 5, 5 over 9 -- 75 taps per output instead of 275.
void Plan::chainMaxPools()
{
    const auto eligible = [&](const PlanOp &op) {
        return !op.dead && op.kind == PlanOp::MAXPOOL && op.stride == 1 && op.ksize % 2 == 1 && op.pad == op.ksize / 2;
    };
    std::vector<bool> done(ops.size(), false);
    for (size_t i = 0; i < ops.size(); ++i)
    {
        if (done[i] || !eligible(ops[i])) continue;
        std::vector<size_t> slots;
        for (size_t j = i; j < ops.size(); ++j)
            if (!done[j] && eligible(ops[j]) && ops[j].in0 == ops[i].in0) { slots.push_back(j); done[j] = true; }
        if (slots.size() < 2) continue;
        // the members change places inside their own slots only; nothing between them may read one of them, and with
        // per-layer outputs kept (pinned) every member must belong to the same layer, whose ops run as one unit
        bool ok = true;
        for (size_t k = slots.front(); k <= slots.back() && ok; ++k)
        {
            if (std::find(slots.begin(), slots.end(), k) != slots.end() || ops[k].dead) continue;
            for (size_t m : slots)
                if (ops[k].in0 == ops[m].out || ops[k].in1 == ops[m].out) ok = false;
        }
        for (size_t m : slots)
        {
            if (ops[m].layerIndex != ops[slots.front()].layerIndex && (tensors[static_cast<size_t>(ops[m].out)].pinned || tensors[static_cast<size_t>(ops[slots.front()].out)].pinned)) ok = false;
            for (size_t m2 : slots)
                if (m2 != m && ops[m2].ksize == ops[m].ksize) ok = false;
        }
        if (!ok) continue;
        std::vector<size_t> byK(slots);
        std::sort(byK.begin(), byK.end(), [&](size_t a, size_t b) { return ops[a].ksize < ops[b].ksize; });
        std::vector<PlanOp> moved;
        for (size_t m : byK) moved.push_back(std::move(ops[m]));
        for (size_t q = 0; q < slots.size(); ++q) ops[slots[q]] = std::move(moved[q]);
        int prevK = ops[slots[0]].ksize;
        for (size_t q = 1; q < slots.size(); ++q)
        {
            PlanOp &cur = ops[slots[q]];
            const int k = cur.ksize;
            cur.in0 = ops[slots[q - 1]].out;
            cur.ksize = k - prevK + 1;
            cur.pad = cur.ksize / 2;
            prevK = k;
        }
        // pools of one window size over one tile that fits LDS run as ONE launch, issued where the first of them stands
        // (msnh_hip_maxpool_chain): the others keep their place in the op list -- their outputs, lifetimes and calibration
        // stay what they are -- but launch nothing
        bool sameK = slots.size() <= 3;
        for (size_t q = 1; q < slots.size(); ++q) sameK = sameK && ops[slots[q]].ksize == ops[slots[0]].ksize;
        const PlanTensor &in = tensors[static_cast<size_t>(ops[slots[0]].in0)];
        if (sameK && in.layout == PlanTensor::NHWC && !std::getenv("MSNH_NO_POOL_CHAIN") &&
            msnh_hip_maxpool_chain_supported(in.dtype, in.h, in.w, in.c, ops[slots[0]].ksize, static_cast<int>(slots.size())))
            for (size_t q = 1; q < slots.size(); ++q)
            {
                ops[slots[q]].chainHead = static_cast<int>(slots[0]);
                ops[slots[q - 1]].chainNext = static_cast<int>(slots[q]);
            }
    }
}

// ---- pass 2: concat aliasing ---------------------------------------------------------------------------------------
void Plan::aliasConcats()
{
    for (size_t i = 0; i < ops.size(); ++i)
    {
        PlanOp &cp = ops[i];
        if (cp.dead || cp.kind != PlanOp::COPY) continue;
        PlanTensor &src = tensors[static_cast<size_t>(cp.in0)];
        const PlanTensor &dst = tensors[static_cast<size_t>(cp.out)];
        if (src.parent >= 0 || src.external || src.layout != PlanTensor::NHWC || dst.layout != PlanTensor::NHWC) continue;
        if (src.dtype != dst.dtype) continue;
        if (cp.dstChanOffset % 8 != 0 || dst.c % 8 != 0 || src.c % 8 != 0) continue;     // keep 16-byte alignment for vector kernels
        if (root(cp.out) == cp.in0) continue;
        bool ok = true;
        for (const PlanOp &op : ops)
        {
            if (op.dead) continue;
            const bool reads = op.in0 == cp.in0 || op.in1 == cp.in0;
            if (reads && op.kind == PlanOp::CONNECTED) ok = false;          // needs densely packed rows
        }
        const int p = producerOf(cp.in0);
        if (p < 0 || static_cast<size_t>(p) > i) ok = false;
        if (!ok) continue;
        src.parent = cp.out;
        src.chanOffset = cp.dstChanOffset;
        cp.dead = true;
    }
}

// ---- pass 3: calibration -------------------------------------------------------------------------------------------
// Runs the plan once and takes max|x| of every tensor right behind the launch that writes it.  (Measuring after the whole forward
// would read arena space that later tensors have reused: a tensor of the first layers would then be given the magnitude of whatever
// ended up in its place, and with it a scale that flushes its own values to zero.)
void Plan::runCalibration(msnh_stream_t s)
{
    struct WriteAll { bool &f; explicit WriteAll(bool &x) : f(x) { f = true; } ~WriteAll() { f = false; } } writeAll(_tailWriteAll);
    DeviceBuffer res(sizeof(float) * tensors.size());
    MSNH_DEV(msnh_hip_fill_zero(res.ptr(), sizeof(float) * tensors.size(), s));
    for (PlanOp &op : ops)
    {
        if (op.dead) continue;
        launch(op, s);
        if (op.out < 0) continue;
        const PlanTensor &pt = tensors[static_cast<size_t>(op.out)];
        if (pt.layout != PlanTensor::NHWC) continue;
        if (op.kind == PlanOp::COPY)
        {
            // a copy fills a channel slice of its output; the other slices may not have been written yet
            const size_t el = pt.dtype == MSNH_F16 ? 2 : 4;
            const void *slice = static_cast<const unsigned char *>(ptr(op.out)) + static_cast<size_t>(op.dstChanOffset) * el;
            MSNH_DEV(msnh_hip_absmax(pt.dtype, pt.pixels(), tensors[static_cast<size_t>(op.in0)].c, slice, ld(op.out), res.as<float>() + op.out, s));
            continue;
        }
        MSNH_DEV(msnh_hip_absmax(pt.dtype, pt.pixels(), pt.c, ptr(op.out), ld(op.out), res.as<float>() + op.out, s));
    }
    std::vector<float> host(tensors.size(), 0.f);
    MSNH_DEV(msnh_hip_memcpy_d2h(host.data(), res.ptr(), sizeof(float) * tensors.size(), s));
    MSNH_DEV(msnh_hip_stream_sync(s));
    for (size_t t = 0; t < tensors.size(); ++t) tensors[t].amax = host[t];
}

// Eager run on the current input; for every float16 tensor the largest stored magnitude and the number of non-finite elements.
// Returns 65504 / (largest stored float16 magnitude), 0 if any float16 tensor holds an infinite or NaN element: the factor by which
// the input could still grow before a float16 activation overflows.
float Plan::fp16Headroom(msnh_stream_t s)
{
    struct WriteAll { bool &f; explicit WriteAll(bool &x) : f(x) { f = true; } ~WriteAll() { f = false; } } writeAll(_tailWriteAll);
    DeviceBuffer res(sizeof(float) * 2);
    MSNH_DEV(msnh_hip_fill_zero(res.ptr(), sizeof(float) * 2, s));
    if (yoloCandCnt.ptr()) MSNH_DEV(msnh_hip_fill_zero(yoloCandCnt.ptr(), yoloCandCnt.bytes(), s));
    for (PlanOp &op : ops)
    {
        if (op.dead) continue;
        launch(op, s);
        if (op.out < 0) continue;
        const PlanTensor &pt = tensors[static_cast<size_t>(op.out)];
        if (pt.layout != PlanTensor::NHWC || pt.dtype != MSNH_F16 || op.kind == PlanOp::COPY) continue;
        MSNH_DEV(msnh_hip_absmax(pt.dtype, pt.pixels(), pt.c, ptr(op.out), ld(op.out), res.as<float>(), s));
        MSNH_DEV(msnh_hip_count_nonfinite(pt.dtype, pt.pixels(), pt.c, ptr(op.out), ld(op.out), res.as<unsigned>() + 1, s));
    }
    float host[2] = {0.f, 0.f};
    MSNH_DEV(msnh_hip_memcpy_d2h(host, res.ptr(), sizeof(host), s));
    MSNH_DEV(msnh_hip_stream_sync(s));
    unsigned bad = 0;
    std::memcpy(&bad, &host[1], sizeof(bad));
    if (bad != 0) return 0.f;
    return host[0] > 0.f ? 65504.f / host[0] : std::numeric_limits<float>::infinity();
}

std::vector<float> Plan::amaxOfTensors() const
{
    std::vector<float> a(tensors.size());
    for (size_t t = 0; t < tensors.size(); ++t) a[t] = tensors[t].amax;
    return a;
}

uint64_t Plan::structureHash() const
{
    std::ostringstream os;
    for (const PlanTensor &t : tensors)
        os << t.n << ' ' << t.h << ' ' << t.w << ' ' << t.c << ' ' << t.dtype << ' ' << static_cast<int>(t.layout) << ' ' << t.parent << ' ' << t.chanOffset << ';';
    for (const PlanOp &op : ops)
        os << static_cast<int>(op.kind) << ' ' << op.in0 << ' ' << op.in1 << ' ' << op.out << ' ' << (op.dead && op.tailOf < 0) << ' ' << op.layerIndex << ' ' << op.ksize << ' ' << op.stride << ' '
           << op.pad << ' ' << op.dilation << ' ' << op.groups << ' ' << static_cast<int>(op.act) << ' ' << static_cast<int>(op.act2) << ' ' << op.in1Sign << ' ' << (op.src2 != nullptr)
           << ' ' << op.dstChanOffset << ' ' << op.stemOp << ' ' << op.chainHead << ' ' << op.mbExpand << ' ' << op.tail << ' ' << op.stemTail << ' ' << op.up2 << ';';
    const std::string text = os.str();
    return PackFile::hash(text.data(), text.size());
}

void Plan::applyCalibration(const std::vector<float> &calAmax)
{
    if (calAmax.size() != tensors.size()) MSNH_THROW("calibration plan does not match");
    // tensors that must share one scale: views with their parent, pooling / upsample inputs with outputs
    std::vector<int> group(tensors.size());
    std::iota(group.begin(), group.end(), 0);
    std::function<int(int)> find = [&](int x) { return group[static_cast<size_t>(x)] == x ? x : group[static_cast<size_t>(x)] = find(group[static_cast<size_t>(x)]); };
    auto unite = [&](int a, int b) { group[static_cast<size_t>(find(a))] = find(b); };
    for (size_t t = 0; t < tensors.size(); ++t)
        if (tensors[t].parent >= 0) unite(static_cast<int>(t), tensors[t].parent);
    for (const PlanOp &op : ops)
        if (!op.dead && (op.kind == PlanOp::MAXPOOL || op.kind == PlanOp::UPSAMPLE)) unite(op.in0, op.out);
    std::vector<float> gmax(tensors.size(), 0.f);
    for (size_t t = 0; t < tensors.size(); ++t)
    {
        const int g = find(static_cast<int>(t));
        gmax[static_cast<size_t>(g)] = std::max(gmax[static_cast<size_t>(g)], calAmax[t]);
    }
    // Keep the calibrated maximum at or below 2^11: a 32x margin to the half maximum for inputs that run
    // hotter than the calibration image, while staying far above the subnormal range.
    const float target = 2048.f;
    for (size_t t = 0; t < tensors.size(); ++t)
    {
        PlanTensor &pt = tensors[t];
        pt.amax = calAmax[t];
        const float m = gmax[static_cast<size_t>(find(static_cast<int>(t)))];
        pt.scaleExp = 0;
        if (pt.dtype == MSNH_F16 && pt.layout == PlanTensor::NHWC && m > target)
            pt.scaleExp = static_cast<int>(std::ceil(std::log2(m / target)));
    }
    // a float16 tensor sharing a group with a float32 one (possible for maxpool/upsample pairs) keeps exponent 0 on
    // the float32 side only if the whole group is 0; otherwise force the group to 0 is unnecessary because such
    // pairs always share the dtype in the plans this library builds.
}

// ---- pass 4: placement ---------------------------------------------------------------------------------------------
void Plan::place()
{
    const int nT = static_cast<int>(tensors.size());
    const int nOps = static_cast<int>(ops.size());
    std::vector<int> first(static_cast<size_t>(nT), std::numeric_limits<int>::max()), last(static_cast<size_t>(nT), -1);
    auto touch = [&](int t, int i) {
        if (t < 0) return;
        const int r = root(t);
        first[static_cast<size_t>(r)] = std::min(first[static_cast<size_t>(r)], i);
        last[static_cast<size_t>(r)] = std::max(last[static_cast<size_t>(r)], i);
    };
    for (int i = 0; i < nOps; ++i)
    {
        const PlanOp &op = ops[static_cast<size_t>(i)];
        if (op.dead) continue;
        touch(op.in0, i); touch(op.in1, i); touch(op.out, i);
        if (op.chainHead >= 0) touch(op.out, op.chainHead);      // written by the launch of the chain's first pool
        if (op.tail >= 0) touch(ops[static_cast<size_t>(op.tail)].out, i);   // may be written by this launch (msnh_hip_conv2d_tail)
        if (op.stemTail >= 0) touch(ops[static_cast<size_t>(op.stemTail)].out, i);   // written by this launch (msnh_hip_conv_stem_down_tail)
    }
    {
        // the heads of a detector may all be decoded by one launch where the last of them stands (findYoloHeads): their inputs
        // stay alive until then
        int lastHead = -1;
        for (int i = 0; i < nOps; ++i)
            if (!ops[static_cast<size_t>(i)].dead && ops[static_cast<size_t>(i)].kind == PlanOp::YOLO_DECODE) lastHead = i;
        for (int i = 0; i < lastHead; ++i)
            if (!ops[static_cast<size_t>(i)].dead && ops[static_cast<size_t>(i)].kind == PlanOp::YOLO_DECODE) touch(ops[static_cast<size_t>(i)].in0, lastHead);
    }
    for (int t = 0; t < nT; ++t)
    {
        if (!tensors[static_cast<size_t>(t)].persistent && !tensors[static_cast<size_t>(t)].pinned) continue;
        const int r = root(t);
        if (last[static_cast<size_t>(r)] >= 0 && tensors[static_cast<size_t>(t)].persistent) last[static_cast<size_t>(r)] = nOps;
    }
    struct Item { int t; size_t bytes; int first, last; size_t offset; };
    std::vector<Item> items;
    for (int t = 0; t < nT; ++t)
    {
        PlanTensor &pt = tensors[static_cast<size_t>(t)];
        if (pt.parent >= 0) continue;
        if (pt.layout == PlanTensor::NHWC) pt.ld = (pt.c + 7) / 8 * 8;
        else pt.ld = pt.c;
        if (pt.external || last[static_cast<size_t>(t)] < 0) continue;
        const size_t el = pt.dtype == MSNH_F16 ? 2 : 4;
        size_t bytes = static_cast<size_t>(pt.n) * pt.h * pt.w * pt.ld * el;
        bytes = (bytes + 255) / 256 * 256;
        pt.bytes = bytes;
        items.push_back({t, bytes, first[static_cast<size_t>(t)], last[static_cast<size_t>(t)], 0});
    }
    std::sort(items.begin(), items.end(), [](const Item &a, const Item &b) { return a.first != b.first ? a.first < b.first : a.bytes > b.bytes; });
    std::vector<Item> placed;
    size_t total = 0;
    for (Item &it : items)
    {
        // gaps between the tensors alive at the same time, lowest offset first
        std::vector<std::pair<size_t, size_t>> busy;
        for (const Item &p : placed)
            if (!(p.last < it.first || p.first > it.last)) busy.emplace_back(p.offset, p.offset + p.bytes);
        std::sort(busy.begin(), busy.end());
        size_t at = 0;
        for (const auto &b : busy)
        {
            if (at + it.bytes <= b.first) break;
            at = std::max(at, b.second);
        }
        it.offset = at;
        tensors[static_cast<size_t>(it.t)].offset = at;
        total = std::max(total, at + it.bytes);
        placed.push_back(it);
    }
    _arena.alloc(std::max<size_t>(total, 256));
}

// ---- weights -------------------------------------------------------------------------------------------------------
static msnh_conv_desc convDesc(const Plan &plan, const PlanOp &op)
{
    const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
    const PlanTensor &out = plan.tensors[static_cast<size_t>(op.out)];
    msnh_conv_desc d;
    std::memset(&d, 0, sizeof(d));
    const bool fromInput = in.layout == PlanTensor::NCHW_INPUT;
    d.dtype = fromInput ? out.dtype : in.dtype;
    d.out_dtype = out.dtype;
    d.batch = in.n; d.in_h = in.h; d.in_w = in.w; d.in_c = in.c;
    d.in_ld = fromInput ? in.c : plan.ld(op.in0);
    d.out_c = out.c; d.out_h = out.h; d.out_w = out.w; d.out_ld = plan.ld(op.out);
    d.ksize = op.ksize; d.stride = op.stride; d.pad = op.pad; d.dilation = op.dilation; d.groups = op.groups;
    d.act = static_cast<int>(op.act); d.act_param = op.actParam;
    d.has_residual = op.in1 >= 0 ? 1 : 0;
    d.res_ld = op.in1 >= 0 ? plan.ld(op.in1) : out.c;
    d.act2 = static_cast<int>(op.act2); d.act2_param = op.act2Param;
    d.res_mul = op.in1 >= 0 ? op.in1Sign * plan.mulOf(op.in1) : 1.f;
    d.out_mul = 1.f / plan.mulOf(op.out);
    d.algo = op.algo;
    d.tile = op.tile;
    if (op.up2) { d.out_h = out.h / 2; d.out_w = out.w / 2; d.out_upsample = 2; }
    return d;
}

static msnh_mbconv_desc mbconvDesc(const Plan &plan, const PlanOp &op)
{
    const PlanOp &ex = plan.ops[static_cast<size_t>(op.mbExpand)];
    const PlanOp &dw = plan.ops[static_cast<size_t>(op.mbDw)];
    const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
    const PlanTensor &wide = plan.tensors[static_cast<size_t>(ex.out)];
    const PlanTensor &out = plan.tensors[static_cast<size_t>(op.out)];
    msnh_mbconv_desc d;
    std::memset(&d, 0, sizeof(d));
    d.batch = in.n; d.in_h = in.h; d.in_w = in.w; d.in_c = in.c; d.in_ld = plan.ld(op.in0);
    d.exp_c = wide.c; d.stride = dw.stride;
    d.out_c = out.c; d.out_h = out.h; d.out_w = out.w; d.out_ld = plan.ld(op.out);
    d.act1 = static_cast<int>(ex.act); d.act2 = static_cast<int>(dw.act); d.act3 = static_cast<int>(op.act); d.act4 = static_cast<int>(op.act2);
    d.act1_param = ex.actParam; d.act2_param = dw.actParam; d.act3_param = op.actParam; d.act4_param = op.act2Param;
    d.has_residual = op.in1 >= 0 ? 1 : 0;
    d.res_ld = op.in1 >= 0 ? plan.ld(op.in1) : out.c;
    d.mul1 = 1.f / plan.mulOf(ex.out);
    d.mul2 = 1.f / plan.mulOf(dw.out);
    d.out_mul = 1.f / plan.mulOf(op.out);
    d.res_mul = op.in1 >= 0 ? op.in1Sign * plan.mulOf(op.in1) : 1.f;
    return d;
}

// folded affine of a convolution op (its own bias / batch-norm, a batch-norm layer fused behind it, the power-of-two scale of its input);
// empty vectors mean 1 and 0
static void foldAffine(const PlanOp &o, int channels, float inMul, std::vector<float> &scale, std::vector<float> &shift)
{
    scale.clear(); shift.clear();
    o.src->foldedAffine(scale, shift);
    if (o.src2)
    {
        std::vector<float> s2, h2;
        o.src2->foldedAffine(s2, h2);
        if (scale.empty()) scale.assign(static_cast<size_t>(channels), 1.f);
        if (shift.empty()) shift.assign(static_cast<size_t>(channels), 0.f);
        for (size_t c = 0; c < static_cast<size_t>(channels); ++c) { scale[c] = s2[c] * scale[c]; shift[c] = s2[c] * shift[c] + h2[c]; }
    }
    if (inMul != 1.f)
    {
        if (scale.empty()) scale.assign(static_cast<size_t>(channels), 1.f);
        for (float &v : scale) v *= inMul;
    }
}

static std::vector<uint16_t> toHalf(const std::vector<float> &v);

void Plan::prepareWeights(PackFile *from, PackFile *to)
{
    size_t workspace = 0;
    for (size_t opIndex = 0; opIndex < ops.size(); ++opIndex)
    {
        PlanOp &op = ops[opIndex];
        if (op.dead) continue;
        if (op.kind == PlanOp::CONV && op.stemOp >= 0)
        {
            // the fused pair: both kernels packed into MFMA lane order, both batch-norms folded; the second layer's scale undoes the
            // power-of-two scale of the values the first layer leaves in LDS
            const PlanOp &first = ops[static_cast<size_t>(op.stemOp)];
            const PlanTensor &mid = tensors[static_cast<size_t>(first.out)];
            const PlanTensor &out = tensors[static_cast<size_t>(op.out)];
            const std::vector<float> &w1 = first.src->kernelWeights(), &w2 = op.src->kernelWeights();
            if (w1.size() != static_cast<size_t>(mid.c) * 27 || w2.size() != static_cast<size_t>(out.c) * mid.c * 9) MSNH_THROW("conv weights are not loaded (" + op.name + ")");
            std::vector<uint16_t> p1(msnh_hip_conv_stem_down_packed_elems(out.c, 0)), p2(msnh_hip_conv_stem_down_packed_elems(out.c, 1));
            MSNH_DEV(msnh_hip_conv_stem_down_pack(w1.data(), out.c, w2.data(), p1.data(), p2.data()));
            op.wDev2.upload(p1.data(), p1.size() * 2);
            op.wDev.upload(p2.data(), p2.size() * 2);
            const auto affine = [&](const PlanOp &o, int channels, float inMul, DeviceBuffer &scaleDev, DeviceBuffer &shiftDev) {
                std::vector<float> scale, shift;
                o.src->foldedAffine(scale, shift);
                if (o.src2)
                {
                    std::vector<float> s2, h2;
                    o.src2->foldedAffine(s2, h2);
                    if (scale.empty()) scale.assign(static_cast<size_t>(channels), 1.f);
                    if (shift.empty()) shift.assign(static_cast<size_t>(channels), 0.f);
                    for (size_t c = 0; c < static_cast<size_t>(channels); ++c) { scale[c] = s2[c] * scale[c]; shift[c] = s2[c] * shift[c] + h2[c]; }
                }
                if (inMul != 1.f)
                {
                    if (scale.empty()) scale.assign(static_cast<size_t>(channels), 1.f);
                    for (float &v : scale) v *= inMul;
                }
                if (!scale.empty()) scaleDev.upload(scale.data(), scale.size() * sizeof(float));
                if (!shift.empty()) shiftDev.upload(shift.data(), shift.size() * sizeof(float));
            };
            affine(first, mid.c, 1.f, op.scaleDev2, op.shiftDev2);
            affine(op, out.c, mulOf(first.out), op.scaleDev, op.shiftDev);
            op.algo = MSNH_CONV_STEM_DOWN;
            const PlanTensor &img = tensors[static_cast<size_t>(op.in0)];
            op.flops = 2.0 * img.n * (static_cast<double>(mid.c) * mid.h * mid.w * img.c * 9 + static_cast<double>(out.c) * out.h * out.w * mid.c * 9);
            if (op.stemTail >= 0)
            {
                const PlanOp &tail = ops[static_cast<size_t>(op.stemTail)];
                const PlanTensor &z = tensors[static_cast<size_t>(tail.out)];
                const std::vector<float> &w3 = tail.src->kernelWeights();
                if (w3.size() != static_cast<size_t>(z.c) * out.c) MSNH_THROW("conv weights are not loaded (" + tail.name + ")");
                std::vector<uint16_t> p3(msnh_hip_conv_stem_down_tail_packed_elems(out.c));
                MSNH_DEV(msnh_hip_conv_stem_down_tail_pack(out.c, w3.data(), p3.data()));
                op.wDev3.upload(p3.data(), p3.size() * 2);
                affine(tail, z.c, mulOf(op.out), op.scaleDev3, op.shiftDev3);
                op.flops += 2.0 * img.n * static_cast<double>(z.c) * z.h * z.w * out.c;
            }
            continue;
        }
        if (op.kind == PlanOp::CONV && op.mbExpand >= 0)
        {
            // the fused inverted-residual block: both 1x1 filters in fragment order, the depthwise taps and the first two affines in one
            // packed record per 64 widened channels; each stage's scale undoes the power-of-two scale of the tensor it reads
            const PlanOp &ex = ops[static_cast<size_t>(op.mbExpand)];
            const PlanOp &dw = ops[static_cast<size_t>(op.mbDw)];
            const msnh_mbconv_desc d = mbconvDesc(*this, op);
            const std::vector<float> &w1 = ex.src->kernelWeights(), &w2 = dw.src->kernelWeights(), &w3 = op.src->kernelWeights();
            if (w1.size() != static_cast<size_t>(d.exp_c) * d.in_c || w2.size() != static_cast<size_t>(d.exp_c) * 9 || w3.size() != static_cast<size_t>(d.out_c) * d.exp_c)
                MSNH_THROW("conv weights are not loaded (" + op.name + ")");
            std::vector<float> s1, h1, s2, h2, s3, h3;
            foldAffine(ex, d.exp_c, mulOf(op.in0), s1, h1);
            foldAffine(dw, d.exp_c, mulOf(ex.out), s2, h2);
            foldAffine(op, d.out_c, mulOf(dw.out), s3, h3);
            std::vector<unsigned char> packed(msnh_hip_mbconv_packed_bytes(&d));
            if (packed.empty()) MSNH_THROW("mbconv: the block is not supported after placement (" + op.name + ")");
            MSNH_DEV(msnh_hip_mbconv_pack(&d, w1.data(), s1.empty() ? nullptr : s1.data(), h1.empty() ? nullptr : h1.data(), w2.data(), s2.empty() ? nullptr : s2.data(),
                                          h2.empty() ? nullptr : h2.data(), w3.data(), packed.data()));
            op.wDev.upload(packed.data(), packed.size());
            if (!s3.empty()) op.scaleDev.upload(s3.data(), s3.size() * sizeof(float));
            if (!h3.empty()) op.shiftDev.upload(h3.data(), h3.size() * sizeof(float));
            op.algo = MSNH_CONV_MBCONV;
            const PlanTensor &wide = tensors[static_cast<size_t>(ex.out)];
            const PlanTensor &narrow = tensors[static_cast<size_t>(dw.out)];
            op.flops = 2.0 * d.batch * (static_cast<double>(wide.h) * wide.w * d.exp_c * d.in_c + static_cast<double>(narrow.h) * narrow.w * d.exp_c * 9 +
                                        static_cast<double>(d.out_h) * d.out_w * d.out_c * d.exp_c);
            continue;
        }
        if (op.kind == PlanOp::CONV)
        {
            const PlanTensor &in = tensors[static_cast<size_t>(op.in0)];
            msnh_conv_desc d = convDesc(*this, op);
            if (in.layout == PlanTensor::NCHW_INPUT) d.algo = MSNH_CONV_STEM;
            op.algo = msnh_hip_conv2d_select_algo(&d);
            if (op.algo == MSNH_CONV_STEM && in.layout != PlanTensor::NCHW_INPUT)
            {
                // the first-layer kernel reads the network's NCHW float32 input; a few-channel image tensor made on the device (a
                // padding or slice layer in front of the first convolution) is NHWC like every other
                msnh_conv_desc nd = d;
                nd.algo = MSNH_CONV_IGEMM;
                op.algo = msnh_hip_conv2d_tile_supported(&nd, 0) ? MSNH_CONV_IGEMM : MSNH_CONV_DIRECT;
            }
            if (preferWinograd && op.algo == MSNH_CONV_IGEMM)
            {
                msnh_conv_desc wd = d;
                wd.algo = MSNH_CONV_WINOGRAD;
                if (msnh_hip_conv2d_tile_supported(&wd, 0)) op.algo = MSNH_CONV_WINOGRAD;
            }
            d.algo = op.algo;
            workspace = std::max(workspace, msnh_hip_conv2d_workspace_bytes(&d, op.algo));
            const std::vector<float> &w = op.src->kernelWeights();
            const size_t expect = static_cast<size_t>(d.out_c) * (d.in_c / d.groups) * d.ksize * d.ksize;
            if (w.size() != expect) MSNH_THROW("conv weights are not loaded (" + op.name + ")");
            const size_t elems = msnh_hip_conv2d_packed_weight_elems(&d, op.algo);
            const size_t el = d.dtype == MSNH_F16 ? 2 : 4;
            const unsigned char *kept = from ? from->blob(static_cast<uint32_t>(opIndex), static_cast<uint32_t>(op.algo), elems * el) : nullptr;
            if (kept) op.wDev.upload(kept, elems * el);
            else
            {
                std::vector<unsigned char> packed(elems * el);
                MSNH_DEV(msnh_hip_conv2d_pack_weights(&d, op.algo, w.data(), packed.data()));
                op.wDev.upload(packed.data(), packed.size());
                if (to) to->add(static_cast<uint32_t>(opIndex), static_cast<uint32_t>(op.algo), packed.data(), packed.size());
            }

            std::vector<float> scale, shift;
            op.src->foldedAffine(scale, shift);
            if (op.src2)
            {
                std::vector<float> s2, h2;
                op.src2->foldedAffine(s2, h2);
                if (scale.empty()) scale.assign(static_cast<size_t>(d.out_c), 1.f);
                if (shift.empty()) shift.assign(static_cast<size_t>(d.out_c), 0.f);
                for (int c = 0; c < d.out_c; ++c)
                {
                    const size_t i = static_cast<size_t>(c);
                    scale[i] = s2[i] * scale[i];
                    shift[i] = s2[i] * shift[i] + h2[i];
                }
            }
            const float inMul = in.layout == PlanTensor::NCHW_INPUT ? 1.f : mulOf(op.in0);
            if (inMul != 1.f)
            {
                if (scale.empty()) scale.assign(static_cast<size_t>(d.out_c), 1.f);
                for (float &v : scale) v *= inMul;
            }
            if (!scale.empty()) op.scaleDev.upload(scale.data(), scale.size() * sizeof(float));
            if (!shift.empty()) op.shiftDev.upload(shift.data(), shift.size() * sizeof(float));
            op.flops = 2.0 * d.batch * d.out_c * d.out_h * d.out_w * (d.in_c / d.groups) * d.ksize * d.ksize;
        }
        else if (op.kind == PlanOp::COL2IM)
        {
            std::vector<float> scale, shift;
            op.src->foldedAffine(scale, shift);
            if (!shift.empty()) op.shiftDev.upload(shift.data(), shift.size() * sizeof(float));
        }
        else if (op.kind == PlanOp::AFFINE)
        {
            std::vector<float> scale, shift;
            op.src->foldedAffine(scale, shift);
            const float inMul = mulOf(op.in0);
            for (float &v : scale) v *= inMul;
            op.scaleDev.upload(scale.data(), scale.size() * sizeof(float));
            op.shiftDev.upload(shift.data(), shift.size() * sizeof(float));
        }
        else if (op.kind == PlanOp::CONNECTED)
        {
            const PlanTensor &in = tensors[static_cast<size_t>(op.in0)];
            const std::vector<float> &w0 = op.src->kernelWeights();
            if (w0.empty()) MSNH_THROW("connected weights are not loaded (" + op.name + ")");
            // The reference flattens an image tensor channel-major, input index = (ch * H + y) * W + x
            // (src/layers/MsnhConnectedLayer.cpp:187 on an NCHW buffer); on the device the pixel's channels are contiguous.
            std::vector<float> permuted;
            const int hw = in.layout == PlanTensor::NHWC ? in.h * in.w : 1;
            // (the record's algorithm field of a connected launch: 100 + dtype + 10 if the weights were permuted to pixel-major)
            const uint32_t packKind = 100u + static_cast<uint32_t>(in.dtype) + (hw > 1 ? 10u : 0u);
            const size_t packBytes = w0.size() * (in.dtype == MSNH_F16 ? 2u : 4u);
            const unsigned char *kept = from ? from->blob(static_cast<uint32_t>(opIndex), packKind, packBytes) : nullptr;
            if (hw > 1 && ld(op.in0) != in.c) MSNH_THROW("connect: an image input needs a channel count that is a multiple of 8 (" + op.name + ")");
            if (hw > 1 && !kept)
            {
                const size_t inputs = static_cast<size_t>(hw) * in.c;
                if (w0.size() % inputs != 0) MSNH_THROW("connect: weight count does not match the input (" + op.name + ")");
                const size_t outputs = w0.size() / inputs;
                permuted.resize(w0.size());
                for (size_t o = 0; o < outputs; ++o)
                    for (int ch = 0; ch < in.c; ++ch)
                        for (int p = 0; p < hw; ++p)
                            permuted[o * inputs + static_cast<size_t>(p) * in.c + ch] = w0[o * inputs + static_cast<size_t>(ch) * hw + p];
            }
            const std::vector<float> &w = hw > 1 && !kept ? permuted : w0;
            if (kept) op.wDev.upload(kept, packBytes);
            else if (in.dtype == MSNH_F16)
            {
                const std::vector<uint16_t> h = toHalf(w);
                op.wDev.upload(h.data(), h.size() * 2);
                if (to) to->add(static_cast<uint32_t>(opIndex), packKind, h.data(), h.size() * 2);
            }
            else
            {
                op.wDev.upload(w.data(), w.size() * sizeof(float));
                if (to) to->add(static_cast<uint32_t>(opIndex), packKind, w.data(), w.size() * sizeof(float));
            }
            std::vector<float> scale, shift;
            op.src->foldedAffine(scale, shift);
            if (!shift.empty()) op.shiftDev.upload(shift.data(), shift.size() * sizeof(float));
            op.flops = 2.0 * static_cast<double>(w.size()) * in.n;
            // a real batch is a GEMM: run it as the 1x1 convolution of a 1x1 image, so that the tile search (and its
            // split-K variant, which suits the few output tiles of a classifier) covers it
            const int vec = in.dtype == MSNH_F16 ? 8 : 4;
            op.algo = MSNH_CONV_AUTO;
            if (in.n >= 8 && in.h * in.w == 1 && in.c % vec == 0 && ld(op.in0) % vec == 0 && mulOf(op.in0) == 1.f && !shift.empty())
            {
                op.ksize = 1; op.stride = 1; op.pad = 0; op.dilation = 1; op.groups = 1;
                op.algo = MSNH_CONV_IGEMM;
                op.tile = in.n <= 64 ? 12 : 0;
            }
        }
    }
    if (workspace > _convWorkspace.bytes()) _convWorkspace.alloc(workspace);
}

// Tune cache, one line per tuned launch: what identifies the launch (shape, dtype, epilogue kind) and what the search chose for it.
static std::string tuneSignature(const Plan &plan, const PlanOp &op)
{
    const PlanTensor &in = plan.tensors[static_cast<size_t>(op.in0)];
    const PlanTensor &out = plan.tensors[static_cast<size_t>(op.out)];
    std::ostringstream os;
    os << static_cast<int>(op.kind) << ' ' << in.n << ' ' << in.h << ' ' << in.w << ' ' << in.c << ' ' << plan.ld(op.in0) << ' ' << out.c << ' '
       << plan.ld(op.out) << ' ' << op.ksize << ' ' << op.stride << ' ' << op.pad << ' ' << op.dilation << ' ' << op.groups << ' ' << (op.in1 >= 0) << ' '
       << in.dtype << ' ' << out.dtype;
    if (op.up2) os << " up2";
    if (op.tail >= 0) os << " tail " << plan.tensors[static_cast<size_t>(plan.ops[static_cast<size_t>(op.tail)].out)].c;
    return os.str();
}

static msnh_conv_tail_desc tailDesc(const Plan &plan, const PlanOp &op)
{
    const PlanOp &b = plan.ops[static_cast<size_t>(op.tail)];
    msnh_conv_tail_desc t;
    std::memset(&t, 0, sizeof(t));
    t.out_c = plan.tensors[static_cast<size_t>(b.out)].c;
    t.out_ld = plan.ld(b.out);
    t.act = static_cast<int>(b.act);
    t.act_param = b.actParam;
    t.out_mul = 1.f / plan.mulOf(b.out);
    t.write_y = op.tailSkipY ? 0 : 1;
    return t;
}

// The choice between one launch and two is the first op's algorithm; the 1x1 op follows it.
void Plan::applyTails()
{
    for (PlanOp &a : ops)
    {
        if (a.tail < 0) continue;
        PlanOp &b = ops[static_cast<size_t>(a.tail)];
        if (a.ownFlops == 0) a.ownFlops = a.flops;
        const bool fused = !a.dead && a.algo == MSNH_CONV_IGEMM_TAIL;
        b.dead = fused;
        a.flops = a.ownFlops + (fused ? b.flops : 0.0);
        // the first convolution's own result stays on the chip when the 1x1 is its only reader: a plain tensor (no view of or into
        // another), not kept for the caller, read by no other live op
        const PlanTensor &y = tensors[static_cast<size_t>(a.out)];
        bool alone = fused && y.parent < 0 && !y.pinned && !y.persistent && !y.external && consumerCount(a.out) == 0;
        for (size_t t = 0; alone && t < tensors.size(); ++t)
            if (tensors[t].parent == a.out) alone = false;
        for (size_t t = 0; alone && t < layerOut.size(); ++t)
            if (layerOut[t] == a.out && t + 1 == layerOut.size()) alone = false;
        a.tailSkipY = alone;
    }
}

static std::string tuneHeader(int nTiles, bool preferWinograd)
{
    char name[256] = {0};
    int cus = 0;
    size_t mem = 0;
    msnh_hip_device_name(name, sizeof(name), &cus, &mem);
    std::string dev(name);
    for (char &ch : dev)
        if (ch == ' ' || ch == '\n') ch = '_';
    // the weights are packed for the algorithm family chosen before the search (Winograd or not), so a file written under the other
    // preference must not be applied
    return "msnhtune 2 " + (dev.empty() ? std::string("device") : dev) + " cus " + std::to_string(cus) + " tiles " + std::to_string(nTiles) + " winograd " +
           std::to_string(preferWinograd ? 1 : 0);
}

// Per-layer search over the implicit-GEMM tile configurations: each candidate runs the real launch (same buffers,
// same epilogue) a few times between two device events; the fastest wins.  Tiles change the result by nothing but the
// float32 summation order, and so does the split-K variant tried for layers with few output tiles.
// With a cache file: a file written by an earlier search over the same launches on the same device replaces the search.
void Plan::tuneConvs(msnh_stream_t s, const std::string &cacheFile)
{
    const int nTiles = msnh_hip_conv2d_tile_count();
    const auto tunable = [](const PlanOp &op) {
        return !op.dead && (op.kind == PlanOp::CONV || op.kind == PlanOp::CONNECTED) && (op.algo == MSNH_CONV_IGEMM || op.algo == MSNH_CONV_WINOGRAD);
    };
    std::vector<size_t> tunedOps;
    for (size_t i = 0; i < ops.size(); ++i)
        if (tunable(ops[i])) tunedOps.push_back(i);
    // A recorded search: header, then "<signature> | <algo> <tile>" per tunable launch in plan order; any mismatch discards it.
    // Two sources: what an earlier load of a plan with the same launches found in this process (instances of one network then run
    // the same kernels and give the same bits), and the cache file beside the weights.
    static std::mutex memoMutex;
    static std::map<std::string, std::string> memoText;
    const std::string memoKey = tuneHeader(nTiles, preferWinograd) + " " + std::to_string(structureHash()) + (forceTail ? " tails forced" : "");
    const auto adopt = [&](std::istream &f) -> bool {
        // file: header, then "<signature> | <algo> <tile>" per tunable launch in plan order; any mismatch discards the file
        std::string line;
        std::vector<std::pair<int, int>> picks;
        bool ok = static_cast<bool>(std::getline(f, line)) && line == tuneHeader(nTiles, preferWinograd);
        for (size_t k = 0; ok && k < tunedOps.size(); ++k)
        {
            ok = static_cast<bool>(std::getline(f, line));
            const size_t bar = ok ? line.find(" | ") : std::string::npos;
            ok = ok && bar != std::string::npos && line.substr(0, bar) == tuneSignature(*this, ops[tunedOps[k]]);
            int algo = 0, tile = 0;
            ok = ok && std::sscanf(line.c_str() + bar + 3, "%d %d", &algo, &tile) == 2 && tile >= 0 && tile <= nTiles &&
                 (algo == MSNH_CONV_IGEMM || algo == MSNH_CONV_WINOGRAD || algo == MSNH_CONV_IGEMM_SPLITK || algo == MSNH_CONV_POINTWISE ||
                  (algo == MSNH_CONV_IGEMM_TAIL && ops[tunedOps[k]].tail >= 0));
            if (ok) picks.emplace_back(algo, tile);
        }
        if (ok)
        {
            // the library must still accept every recorded choice; otherwise the defaults come back and the search runs
            std::vector<std::pair<int, int>> before;
            size_t need = 0;
            for (size_t k = 0; k < tunedOps.size(); ++k)
            {
                PlanOp &op = ops[tunedOps[k]];
                before.emplace_back(op.algo, op.tile);
                // the packed weights on the device are laid out for the algorithm resolved at weight preparation: a recorded choice
                // from the other family (Winograd's transformed filters against the tap-major layout) would read them wrongly
                if ((picks[k].first == MSNH_CONV_WINOGRAD) != (op.algo == MSNH_CONV_WINOGRAD)) ok = false;
                op.algo = picks[k].first; op.tile = picks[k].second;
                const msnh_conv_desc d = convDesc(*this, op);
                if (op.algo == MSNH_CONV_IGEMM_TAIL)
                {
                    // one launch for this op and its 1x1 consumer: both were packed for the implicit GEMM
                    const msnh_conv_tail_desc t = tailDesc(*this, op);
                    msnh_conv_desc c = d;
                    c.algo = MSNH_CONV_IGEMM;
                    if (before.back().first != MSNH_CONV_IGEMM || ops[static_cast<size_t>(op.tail)].algo == MSNH_CONV_WINOGRAD || !msnh_hip_conv2d_tail_supported(&c, &t, op.tile)) ok = false;
                    continue;
                }
                if (!msnh_hip_conv2d_tile_supported(&d, op.tile)) ok = false;
                if (op.kind == PlanOp::CONV && op.wDev.bytes() != msnh_hip_conv2d_packed_weight_elems(&d, op.algo) * (d.dtype == MSNH_F16 ? 2u : 4u)) ok = false;
                need = std::max(need, msnh_hip_conv2d_workspace_bytes(&d, op.algo));
            }
            if (ok)
            {
                if (need > _convWorkspace.bytes()) _convWorkspace.alloc(need);
                applyTails();
                return true;
            }
            for (size_t k = 0; k < tunedOps.size(); ++k) { ops[tunedOps[k]].algo = before[k].first; ops[tunedOps[k]].tile = before[k].second; }
        }
        return false;
    };
    if (!cacheFile.empty())
    {
        std::ifstream f(cacheFile);
        if (f.is_open() && adopt(f))
        {
            std::ifstream again(cacheFile);
            std::ostringstream all;
            all << again.rdbuf();
            std::lock_guard<std::mutex> lk(memoMutex);
            memoText[memoKey] = all.str();
            return;
        }
    }
    {
        std::string text;
        {
            std::lock_guard<std::mutex> lk(memoMutex);
            const auto it = memoText.find(memoKey);
            if (it != memoText.end()) text = it->second;
        }
        if (!text.empty())
        {
            std::istringstream f(text);
            if (adopt(f))
            {
                if (!cacheFile.empty())
                {
                    std::ofstream out(cacheFile, std::ios::trunc);
                    if (out.is_open()) out << text;
                }
                return;
            }
        }
    }

    msnh_event_t e0 = nullptr, e1 = nullptr;
    MSNH_DEV(msnh_hip_event_create(&e0));
    MSNH_DEV(msnh_hip_event_create(&e1));
    struct Key { int kind, b, h, w, c, inLd, oc, outLd, k, st, pad, dil, g, res, odt, algo, up; bool operator==(const Key &o) const { return std::memcmp(this, &o, sizeof(Key)) == 0; } };
    std::vector<std::pair<Key, int>> memo;         // identical shapes share one search
    for (PlanOp &op : ops)
    {
        if (op.dead || (op.kind != PlanOp::CONV && op.kind != PlanOp::CONNECTED) || (op.algo != MSNH_CONV_IGEMM && op.algo != MSNH_CONV_WINOGRAD)) continue;
        const PlanTensor &in = tensors[static_cast<size_t>(op.in0)];
        const PlanTensor &out = tensors[static_cast<size_t>(op.out)];
        Key key;
        std::memset(&key, 0, sizeof(key));
        key.kind = static_cast<int>(op.kind);
        key.b = in.n; key.h = in.h; key.w = in.w; key.c = in.c; key.inLd = ld(op.in0); key.oc = out.c; key.outLd = ld(op.out);
        key.k = op.ksize; key.st = op.stride; key.pad = op.pad; key.dil = op.dilation; key.g = op.groups;
        key.res = op.in1 >= 0; key.odt = out.dtype; key.algo = op.algo; key.up = op.up2 ? 1 : 0;
        bool found = false;
        for (const auto &m : memo)
        {
            if (!(m.first == key)) continue;
            // same launch as one searched before: take its result, if the library accepts it for this op as well
            const int wasAlgo = op.algo, wasTile = op.tile;
            op.algo = m.second / 1000; op.tile = m.second % 1000;
            const msnh_conv_desc d = convDesc(*this, op);
            if (msnh_hip_conv2d_tile_supported(&d, op.tile) && msnh_hip_conv2d_workspace_bytes(&d, op.algo) <= _convWorkspace.bytes()) found = true;
            else { op.algo = wasAlgo; op.tile = wasTile; }
            break;
        }
        if (found) continue;
        // Two passes: every candidate is timed over a few launches, then the four fastest are timed again over many more and the
        // best of those wins (a single short timing of a 10-40 us kernel is too noisy to separate candidates a few percent apart).
        struct Cand { float ms; int algo, tile; };
        std::vector<Cand> cands;
        auto timeOne = [&](int algo, int tile, int warm, int reps) {
            op.algo = algo;
            op.tile = tile;
            for (int r = 0; r < warm; ++r) launch(op, s);            // warm-up (also surfaces launch errors for this tile)
            MSNH_DEV(msnh_hip_event_record(e0, s));
            for (int r = 0; r < reps; ++r) launch(op, s);
            MSNH_DEV(msnh_hip_event_record(e1, s));
            MSNH_DEV(msnh_hip_event_sync(e1));
            float ms = 0.f;
            MSNH_DEV(msnh_hip_event_elapsed_ms(e0, e1, &ms));
            return ms / static_cast<float>(reps);
        };
        auto search = [&](int algo) {
            op.algo = algo;
            for (int tile = 0; tile <= nTiles; ++tile)
            {
                op.tile = tile;
                {
                    const msnh_conv_desc probe = convDesc(*this, op);
                    if (!msnh_hip_conv2d_tile_supported(&probe, tile)) continue;
                }
                cands.push_back({timeOne(algo, tile, 1, 3), algo, tile});
            }
        };
        const int baseAlgo = op.algo;
        search(baseAlgo);
        if (baseAlgo == MSNH_CONV_IGEMM)
        {
            // layers with few output tiles: the K loop cut over several workgroups, if its workspace is modest
            op.tile = 0;
            op.algo = baseAlgo;
            const msnh_conv_desc d = convDesc(*this, op);
            const size_t need = msnh_hip_conv2d_workspace_bytes(&d, MSNH_CONV_IGEMM_SPLITK);
            if (out.c % 4 == 0 && need <= (static_cast<size_t>(256) << 20))
            {
                MSNH_DEV(msnh_hip_stream_sync(s));
                if (need > _convWorkspace.bytes()) _convWorkspace.alloc(need);
                search(MSNH_CONV_IGEMM_SPLITK);
            }
        }
        if (baseAlgo == MSNH_CONV_IGEMM && op.kind == PlanOp::CONV) search(MSNH_CONV_POINTWISE);      // (refused by the library unless the shape fits)
        int best = 0, bestAlgo = baseAlgo;
        if (!cands.empty())
        {
            std::sort(cands.begin(), cands.end(), [](const Cand &x, const Cand &y) { return x.ms < y.ms; });
            const size_t finalists = std::min<size_t>(cands.size(), 4);
            float bestMs = std::numeric_limits<float>::max();
            for (size_t i = 0; i < finalists; ++i)
            {
                const float ms = finalists > 1 ? timeOne(cands[i].algo, cands[i].tile, 2, 16) : cands[i].ms;
                if (ms < bestMs) { bestMs = ms; best = cands[i].tile; bestAlgo = cands[i].algo; }
            }
        }
        op.algo = bestAlgo;
        op.tile = best;
        memo.emplace_back(key, bestAlgo * 1000 + best);
    }
    // Pairs marked by fuse (e): the two launches as chosen above, back to back, against one launch on every tile that carries a tail.
    {
        struct PairKey { std::string a, b; int tile; };
        std::vector<PairKey> pairMemo;              // identical pairs share one comparison; tile 0 = two launches
        for (PlanOp &a : ops)
        {
            if (a.dead || a.tail < 0 || a.kind != PlanOp::CONV || a.algo != MSNH_CONV_IGEMM) continue;
            PlanOp &b = ops[static_cast<size_t>(a.tail)];
            if (b.dead || (b.algo != MSNH_CONV_IGEMM && b.algo != MSNH_CONV_POINTWISE)) continue;
            const std::string ka = tuneSignature(*this, a), kb = tuneSignature(*this, b);
            const int twoTile = a.tile;
            bool found = false;
            for (const PairKey &m : pairMemo)
                if (m.a == ka && m.b == kb)
                {
                    if (m.tile > 0) { a.algo = MSNH_CONV_IGEMM_TAIL; a.tile = m.tile; }
                    found = true;
                    break;
                }
            if (found) continue;
            const auto timePair = [&](int reps) {
                for (int r = 0; r < 2; ++r) { launch(a, s); if (a.algo != MSNH_CONV_IGEMM_TAIL) launch(b, s); }
                MSNH_DEV(msnh_hip_event_record(e0, s));
                for (int r = 0; r < reps; ++r) { launch(a, s); if (a.algo != MSNH_CONV_IGEMM_TAIL) launch(b, s); }
                MSNH_DEV(msnh_hip_event_record(e1, s));
                MSNH_DEV(msnh_hip_event_sync(e1));
                float ms = 0.f;
                MSNH_DEV(msnh_hip_event_elapsed_ms(e0, e1, &ms));
                return ms / static_cast<float>(reps);
            };
            // One launch has to win by a margin: timed alone and repeated, the pair's second launch finds its input in the caches more
            // reliably than it does inside a forward, and a tie here was a small loss there.
            float bestMs = timePair(16) * (forceTail ? 1.f : 0.95f);
            int bestTile = 0;
            const msnh_conv_tail_desc t = tailDesc(*this, a);
            for (int tile = msnh_hip_conv2d_tail_tile_first(); tile <= nTiles; ++tile)
            {
                msnh_conv_desc c = convDesc(*this, a);
                c.algo = MSNH_CONV_IGEMM;
                if (!msnh_hip_conv2d_tail_supported(&c, &t, tile)) continue;
                a.algo = MSNH_CONV_IGEMM_TAIL; a.tile = tile;
                const float ms = timePair(16);
                if (ms < bestMs || (forceTail && bestTile == 0)) { bestMs = ms; bestTile = tile; }
            }
            if (bestTile > 0) { a.algo = MSNH_CONV_IGEMM_TAIL; a.tile = bestTile; }
            else { a.algo = MSNH_CONV_IGEMM; a.tile = twoTile; }
            pairMemo.push_back({ka, kb, bestTile});
        }
    }
    applyTails();
    msnh_hip_event_destroy(e0);
    msnh_hip_event_destroy(e1);
    std::ostringstream text;
    text << tuneHeader(nTiles, preferWinograd) << "\n";
    for (size_t i : tunedOps)
    {
        // (the signature is taken with the searched choice in place: it does not depend on algo / tile)
        text << tuneSignature(*this, ops[i]) << " | " << ops[i].algo << ' ' << ops[i].tile << "\n";
    }
    {
        std::lock_guard<std::mutex> lk(memoMutex);
        memoText[memoKey] = text.str();
    }
    if (!cacheFile.empty())
    {
        std::ofstream f(cacheFile, std::ios::trunc);
        if (f.is_open()) f << text.str();
    }
}

// round-to-nearest-even float -> IEEE half, host side
static uint16_t halfBits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return static_cast<uint16_t>(sign | 0x7c00u | ((x & 0x7fffffu) ? 0x200u : 0));
    if (x >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);                 // rounds to >= 65520 -> inf
    if (x < 0x33000001u) return static_cast<uint16_t>(sign);                            // < 2^-25 -> 0
    int exp = static_cast<int>(x >> 23) - 127;
    uint32_t man = (x & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t base;
    if (exp < -14) { shift = 13 + (-14 - exp); base = 0; }
    else { shift = 13; base = static_cast<uint32_t>(exp + 15) << 10; man &= 0x7fffffu; }
    uint32_t h = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (h & 1u))) ++h;
    return static_cast<uint16_t>(sign | (base + h));
}

static std::vector<uint16_t> toHalf(const std::vector<float> &v)
{
    std::vector<uint16_t> h(v.size());
    for (size_t i = 0; i < v.size(); ++i) h[i] = halfBits(v[i]);
    return h;
}

// ---- execution ---------------------------------------------------------------------------------------------------------
void Plan::launch(PlanOp &op, msnh_stream_t s)
{
    const PlanTensor &in = tensors[static_cast<size_t>(op.in0)];
    const PlanTensor &out = tensors[static_cast<size_t>(op.out)];
    switch (op.kind)
    {
    case PlanOp::CONV:
    {
        if (op.stemOp >= 0)
        {
            const PlanOp &first = ops[static_cast<size_t>(op.stemOp)];
            if (op.stemTail >= 0)
            {
                const PlanOp &tail = ops[static_cast<size_t>(op.stemTail)];
                MSNH_DEV(msnh_hip_conv_stem_down_tail(in.n, in.h, in.w, static_cast<const float *>(ptr(op.in0)), op.wDev2.ptr(), op.scaleDev2.as<float>(),
                                                      op.shiftDev2.as<float>(), static_cast<int>(first.act), first.actParam, 1.f / mulOf(first.out), out.c, op.wDev.ptr(),
                                                      op.scaleDev.as<float>(), op.shiftDev.as<float>(), static_cast<int>(op.act), op.actParam, 1.f / mulOf(op.out),
                                                      ptr(op.out), ld(op.out), op.wDev3.ptr(), op.scaleDev3.as<float>(), op.shiftDev3.as<float>(),
                                                      static_cast<int>(tail.act), tail.actParam, 1.f / mulOf(tail.out), ptr(tail.out), ld(tail.out), s));
                break;
            }
            MSNH_DEV(msnh_hip_conv_stem_down(in.n, in.h, in.w, static_cast<const float *>(ptr(op.in0)), op.wDev2.ptr(), op.scaleDev2.as<float>(), op.shiftDev2.as<float>(),
                                             static_cast<int>(first.act), first.actParam, 1.f / mulOf(first.out), out.c, op.wDev.ptr(), op.scaleDev.as<float>(),
                                             op.shiftDev.as<float>(), static_cast<int>(op.act), op.actParam, 1.f / mulOf(op.out), ptr(op.out), ld(op.out), s));
            break;
        }
        if (op.mbExpand >= 0)
        {
            const msnh_mbconv_desc md = mbconvDesc(*this, op);
            if (op.wDev.bytes() != msnh_hip_mbconv_packed_bytes(&md)) MSNH_THROW("mbconv weights on the device do not fit this launch (" + op.name + ")");
            MSNH_DEV(msnh_hip_mbconv(&md, ptr(op.in0), op.wDev.ptr(), op.scaleDev.as<float>(), op.shiftDev.as<float>(), op.in1 >= 0 ? ptr(op.in1) : nullptr, ptr(op.out), s));
            break;
        }
        if (op.algo == MSNH_CONV_IGEMM_TAIL)
        {
            if (op.tail < 0) MSNH_THROW("no 1x1 convolution follows this launch (" + op.name + ")");
            const PlanOp &b = ops[static_cast<size_t>(op.tail)];
            msnh_conv_desc c = convDesc(*this, op);
            c.algo = MSNH_CONV_IGEMM;
            msnh_conv_tail_desc t = tailDesc(*this, op);
            if (_tailWriteAll) t.write_y = 1;
            if (op.wDev.bytes() != msnh_hip_conv2d_packed_weight_elems(&c, MSNH_CONV_IGEMM) * 2u || b.wDev.bytes() != static_cast<size_t>(t.out_c) * c.out_c * 2u)
                MSNH_THROW("conv weights on the device are not packed for the algorithm of this launch (" + op.name + ")");
            MSNH_DEV(msnh_hip_conv2d_tail(&c, &t, ptr(op.in0), op.wDev.ptr(), op.scaleDev.as<float>(), op.shiftDev.as<float>(), op.in1 >= 0 ? ptr(op.in1) : nullptr,
                                          ptr(op.out), b.wDev.ptr(), b.scaleDev.as<float>(), b.shiftDev.as<float>(), ptr(b.out), s));
            break;
        }
        const msnh_conv_desc d = convDesc(*this, op);
        if (op.wDev.bytes() != msnh_hip_conv2d_packed_weight_elems(&d, op.algo) * (d.dtype == MSNH_F16 ? 2u : 4u))
            MSNH_THROW("conv weights on the device are not packed for the algorithm of this launch (" + op.name + ")");
        MSNH_DEV(msnh_hip_conv2d(&d, ptr(op.in0), op.wDev.ptr(), op.scaleDev.as<float>(), op.shiftDev.as<float>(),
                                 op.in1 >= 0 ? ptr(op.in1) : nullptr, ptr(op.out), _convWorkspace.ptr(), _convWorkspace.bytes(), s));
        break;
    }
    case PlanOp::AFFINE:
        MSNH_DEV(msnh_hip_affine_act(in.dtype, out.dtype, in.pixels(), in.c, ptr(op.in0), ld(op.in0), op.scaleDev.as<float>(),
                                     op.shiftDev.as<float>(), static_cast<int>(op.act), op.actParam, 1.f / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::ADD:
        MSNH_DEV(msnh_hip_add_act(in.dtype, in.pixels(), in.c, ptr(op.in0), ld(op.in0), mulOf(op.in0), ptr(op.in1), ld(op.in1), op.in1Sign * mulOf(op.in1),
                                  static_cast<int>(op.act), op.actParam, 1.f / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::COPY:
    {
        const size_t el = out.dtype == MSNH_F16 ? 2 : 4;
        void *dst = static_cast<unsigned char *>(ptr(op.out)) + static_cast<size_t>(op.dstChanOffset) * el;
        MSNH_DEV(msnh_hip_copy_channels(in.dtype, in.pixels(), in.c, ptr(op.in0), ld(op.in0), mulOf(op.in0) / mulOf(op.out), dst, ld(op.out), s));
        break;
    }
    case PlanOp::MAXPOOL:
        if (op.chainHead >= 0) break;                            // done by the launch of the chain's first pool
        if (op.chainNext >= 0)
        {
            void *ys[3] = {ptr(op.out), nullptr, nullptr};
            int lds[3] = {ld(op.out), 0, 0};
            int steps = 1;
            for (int nx = op.chainNext; nx >= 0 && steps < 3; nx = ops[static_cast<size_t>(nx)].chainNext, ++steps)
            {
                ys[steps] = ptr(ops[static_cast<size_t>(nx)].out);
                lds[steps] = ld(ops[static_cast<size_t>(nx)].out);
            }
            MSNH_DEV(msnh_hip_maxpool_chain(in.dtype, in.n, in.h, in.w, in.c, op.ksize, steps, ptr(op.in0), ld(op.in0), ys, lds, s));
            break;
        }
        MSNH_DEV(msnh_hip_maxpool(in.dtype, in.n, in.h, in.w, in.c, ptr(op.in0), ld(op.in0), op.ksize, op.stride, op.pad, out.h, out.w,
                                  ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::AVGPOOL:
        MSNH_DEV(msnh_hip_avgpool(in.dtype, out.dtype, in.n, in.h, in.w, in.c, ptr(op.in0), ld(op.in0), op.ksize, op.stride, op.pad, out.h,
                                  out.w, mulOf(op.in0) / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::UPSAMPLE:
        MSNH_DEV(msnh_hip_upsample_nearest(in.dtype, in.n, in.h, in.w, in.c, ptr(op.in0), ld(op.in0), op.stride, op.upScale, ptr(op.out),
                                           ld(op.out), s));
        break;
    case PlanOp::PAD:
        MSNH_DEV(msnh_hip_pad(in.dtype, in.n, in.h, in.w, in.c, ptr(op.in0), ld(op.in0), op.padTop, op.padLeft, out.h, out.w, mulOf(op.in0) / mulOf(op.out),
                              op.padValue / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::SLICE:
        MSNH_DEV(msnh_hip_slice(in.dtype, in.n, in.h, in.w, ptr(op.in0), ld(op.in0), op.slice[0], op.slice[1], op.slice[2], op.slice[3], op.slice[4],
                                op.slice[5], out.c, out.h, out.w, mulOf(op.in0) / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::COL2IM:
        MSNH_DEV(msnh_hip_deconv_col2im(in.dtype, in.n, in.h, in.w, out.c, op.ksize, op.stride, op.pad, ptr(op.in0), ld(op.in0), mulOf(op.in0),
                                        op.shiftDev.as<float>(), static_cast<int>(op.act), op.actParam, out.h, out.w, 1.f / mulOf(op.out), ptr(op.out),
                                        ld(op.out), s));
        break;
    case PlanOp::SOFTMAX:
        MSNH_DEV(msnh_hip_softmax(in.dtype, in.n, in.h * in.w, in.c, ptr(op.in0), in.layout == PlanTensor::FLAT ? in.c : ld(op.in0), mulOf(op.in0),
                                  op.upScale, ptr(op.out), out.layout == PlanTensor::FLAT ? out.c : ld(op.out), 1.f / mulOf(op.out), s));
        break;
    case PlanOp::BILINEAR:
        MSNH_DEV(msnh_hip_upsample_bilinear(in.dtype, in.n, in.h, in.w, in.c, ptr(op.in0), ld(op.in0), out.h, out.w, op.alignCorners,
                                            mulOf(op.in0) / mulOf(op.out), ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::CONNECTED:
        if (op.algo == MSNH_CONV_IGEMM || op.algo == MSNH_CONV_IGEMM_SPLITK)
        {
            const msnh_conv_desc d = convDesc(*this, op);
            MSNH_DEV(msnh_hip_conv2d(&d, ptr(op.in0), op.wDev.ptr(), nullptr, op.shiftDev.as<float>(), nullptr, ptr(op.out),
                                     _convWorkspace.ptr(), _convWorkspace.bytes(), s));
            break;
        }
        if (ld(op.in0) != in.c && in.n > 1 && in.h * in.w == 1) MSNH_THROW("connected input must be densely packed");
        MSNH_DEV(msnh_hip_connected(in.dtype, in.n, in.h * in.w * in.c, out.c, ptr(op.in0), mulOf(op.in0), op.wDev.ptr(), op.shiftDev.as<float>(),
                                    static_cast<int>(op.act), op.actParam, static_cast<float *>(ptr(op.out)), s));
        break;
    case PlanOp::INPUT_CAST:
        MSNH_DEV(msnh_hip_nchw_to_nhwc(out.dtype, in.n, in.c, in.h, in.w, static_cast<const float *>(ptr(op.in0)), 1.f / mulOf(op.out),
                                       ptr(op.out), ld(op.out), s));
        break;
    case PlanOp::YOLO_DECODE:
    {
        const int per = 5 + op.classes;
        float *decoded = yoloDecoded.as<float>() + static_cast<size_t>(op.cellBase) * per;
        const bool cand = op.confThresh < 1.5f;
        if (sparseYolo && cand && !yoloHeadOps.empty())
        {
            // all heads in one launch, issued where the last of them stands in the plan (nothing between the heads reads their lists)
            size_t last = 0;
            for (size_t i : yoloHeadOps) last = std::max(last, i);
            if (&op != &ops[last]) break;
            msnh_yolo_head heads[4];
            for (size_t k = 0; k < yoloHeadOps.size(); ++k)
            {
                const PlanOp &h = ops[yoloHeadOps[k]];
                const PlanTensor &t = tensors[static_cast<size_t>(h.in0)];
                heads[k].x = ptr(h.in0); heads[k].x_ld = ld(h.in0); heads[k].x_mul = mulOf(h.in0); heads[k].h = t.h; heads[k].w = t.w;
                for (int i = 0; i < 6; ++i) heads[k].anchors[i] = h.anchors[static_cast<size_t>(i)];
                heads[k].ratio = h.ratio; heads[k].cand_base = h.cellBase;
            }
            MSNH_DEV(msnh_hip_yolo_decode_candidates_heads(in.dtype, in.n, op.classes, static_cast<int>(yoloHeadOps.size()), heads, op.yoloVersion,
                                                           yoloKeepDecoded ? yoloDecoded.as<float>() : nullptr, static_cast<long long>(yoloCells) * per,
                                                           op.confThresh, yoloCandIdx.as<int>(), yoloCells, yoloCandCnt.as<int>(), yoloRows.as<float>(), s));
        }
        else if (sparseYolo && cand)
            MSNH_DEV(msnh_hip_yolo_decode_candidates(in.dtype, in.n, in.h, in.w, op.classes, ptr(op.in0), ld(op.in0), mulOf(op.in0), op.anchors.data(),
                                                     op.ratio, op.yoloVersion, yoloKeepDecoded ? decoded : nullptr, static_cast<long long>(yoloCells) * per, op.confThresh,
                                                     yoloCandIdx.as<int>(), yoloCells, op.cellBase, yoloCandCnt.as<int>(), yoloRows.as<float>(), s));
        else
            MSNH_DEV(msnh_hip_yolo_decode(in.dtype, in.n, in.h, in.w, op.classes, ptr(op.in0), ld(op.in0), mulOf(op.in0), op.anchors.data(), op.ratio,
                                          op.yoloVersion, decoded, static_cast<long long>(yoloCells) * per, op.confThresh,
                                          cand ? yoloCandIdx.as<int>() : nullptr, yoloCells, op.cellBase, cand ? yoloCandCnt.as<int>() : nullptr, s));
        break;
    }
    }
}

// One launch can decode all heads when there are at most four, they agree in everything but geometry and anchors, and their cell
// numbers follow one another from 0 (the candidate list numbers the cells of an image head after head).
void Plan::findYoloHeads()
{
    yoloHeadOps.clear();
    if (std::getenv("MSNH_YOLO_HEAD_LAUNCHES")) return;
    std::vector<size_t> heads;
    for (size_t i = 0; i < ops.size(); ++i)
        if (ops[i].kind == PlanOp::YOLO_DECODE && !ops[i].dead) heads.push_back(i);
    if (heads.size() < 2 || heads.size() > 4) return;
    std::sort(heads.begin(), heads.end(), [this](size_t a, size_t b) { return ops[a].cellBase < ops[b].cellBase; });
    const PlanOp &first = ops[heads[0]];
    int cells = 0;
    for (size_t i : heads)
    {
        const PlanOp &h = ops[i];
        const PlanTensor &t = tensors[static_cast<size_t>(h.in0)];
        const PlanTensor &t0 = tensors[static_cast<size_t>(first.in0)];
        if (h.cellBase != cells || h.classes != first.classes || h.yoloVersion != first.yoloVersion || h.confThresh != first.confThresh ||
            h.confThresh >= 1.5f || t.dtype != t0.dtype || t.n != t0.n)
            return;
        cells += 3 * t.h * t.w;
    }
    if (cells != yoloCells) return;
    yoloHeadOps = heads;
}

void Plan::run(size_t opBegin, size_t opEnd, msnh_stream_t s)
{
    for (size_t i = opBegin; i < opEnd && i < ops.size(); ++i)
        if (!ops[i].dead) launch(ops[i], s);
}

void Plan::exportTensor(int t, std::vector<float> &dst, msnh_stream_t s)
{
    const PlanTensor &pt = tensors[static_cast<size_t>(t)];
    dst.resize(pt.elems());
    if (dst.empty()) return;
    if (pt.layout == PlanTensor::FLAT || pt.layout == PlanTensor::NCHW_INPUT)
    {
        MSNH_DEV(msnh_hip_memcpy_d2h(dst.data(), ptr(t), dst.size() * sizeof(float), s));
        MSNH_DEV(msnh_hip_stream_sync(s));
        return;
    }
    if (_exportScratch.bytes() < dst.size() * sizeof(float)) _exportScratch.alloc(dst.size() * sizeof(float));
    MSNH_DEV(msnh_hip_nhwc_to_nchw(pt.dtype, pt.n, pt.c, pt.h, pt.w, ptr(t), ld(t), mulOf(t), _exportScratch.as<float>(), s));
    MSNH_DEV(msnh_hip_memcpy_d2h(dst.data(), _exportScratch.ptr(), dst.size() * sizeof(float), s));
    MSNH_DEV(msnh_hip_stream_sync(s));
}

std::string Plan::describe() const
{
    static const char *kinds[] = {"conv", "affine", "add", "copy", "maxpool", "avgpool", "upsample", "connected", "input_cast", "yolo_decode", "pad", "slice", "bilinear", "softmax", "col2im"};
    static const char *algos[] = {"auto", "direct", "igemm", "depthwise", "winograd", "stem", "igemm_splitk", "pointwise", "stem+down", "winograd_fused", "mbconv", "igemm+1x1"};
    std::ostringstream os;
    os << "plan: " << liveOps() << " launches, " << tensors.size() << " tensors, arena " << _arena.bytes() / (1024.0 * 1024.0) << " MiB, dtype "
       << (computeDtype == MSNH_F16 ? "f16" : "f32") << "\n";
    for (size_t i = 0; i < ops.size(); ++i)
    {
        const PlanOp &op = ops[i];
        if (op.dead) continue;
        const PlanTensor &in = tensors[static_cast<size_t>(op.in0)];
        const PlanTensor &out = tensors[static_cast<size_t>(op.out)];
        os << "  L" << op.layerIndex << " " << kinds[op.kind];
        if (op.kind == PlanOp::CONV)
            os << "[" << algos[op.algo] << (op.stemTail >= 0 ? "+1x1" : "") << (op.tile ? " t" + std::to_string(op.tile) : std::string()) << " k" << op.ksize << " s" << op.stride << " g" << op.groups << (op.in1 >= 0 ? " +res" : "") << (op.src2 ? " +bn" : "") << (op.up2 ? " +up2" : "") << "]";
        if (op.kind == PlanOp::MAXPOOL || op.kind == PlanOp::AVGPOOL)
            os << "[k" << op.ksize << " s" << op.stride << " p" << op.pad << (op.chainHead >= 0 ? " in the launch of the pool before it" : "") << "]";
        os << " " << in.n << "x" << in.h << "x" << in.w << "x" << in.c << " -> " << out.h << "x" << out.w << "x" << out.c
           << (out.dtype == MSNH_F16 ? " f16" : " f32") << " e" << out.scaleExp;
        if (out.parent >= 0) os << " (slice@" << chanOffsetInRoot(op.out) << " of " << tensors[static_cast<size_t>(root(op.out))].c << ")";
        os << "\n";
    }
    return os.str();
}
}
