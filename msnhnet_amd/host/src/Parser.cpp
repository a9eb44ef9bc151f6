// `.msnhnet` / `.msnhbin` readers.  Behaviour follows src/io/MsnhParser.cpp of the reference (key names,
// defaults, block expansion by `size`, negative layer references, error texts for the cases a caller can
// provoke); the implementation is an indentation scanner plus table-driven key handling.
#include "Msnhnet/io/MsnhParser.h"
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <functional>
#include <map>
#include <sstream>

namespace Msnhnet
{
int BaseParams::index = -1;

// ---- ExString -----------------------------------------------------------------------------------------
void ExString::split(std::vector<std::string> &result, const std::string &str, const std::string &cutset)
{
    size_t pos = 0;
    while (pos < str.size())
    {
        const size_t end = str.find_first_of(cutset, pos);
        const size_t stop = end == std::string::npos ? str.size() : end;
        if (stop > pos) result.push_back(str.substr(pos, stop - pos));
        pos = stop + 1;
    }
}

std::string ExString::trim(const std::string &str)
{
    const size_t a = str.find_first_not_of(" \t\r\n");
    if (a == std::string::npos) return "";
    const size_t b = str.find_last_not_of(" \t\r\n");
    return str.substr(a, b - a + 1);
}

bool ExString::isNumber(const std::string &s)
{
    // [-+]?[0-9]*.?[0-9]+([eE][-+]?[0-9]+)?   ('.' is "any character" in the reference's pattern)
    size_t i = 0;
    const size_t n = s.size();
    if (i < n && (s[i] == '-' || s[i] == '+')) ++i;
    // try every split point for the optional "any char" between the two digit runs
    auto digits = [&](size_t from) { size_t j = from; while (j < n && s[j] >= '0' && s[j] <= '9') ++j; return j; };
    auto tail = [&](size_t j) {
        if (j == n) return true;
        if (s[j] != 'e' && s[j] != 'E') return false;
        ++j;
        if (j < n && (s[j] == '-' || s[j] == '+')) ++j;
        const size_t k = digits(j);
        return k > j && k == n;
    };
    const size_t d1 = digits(i);
    for (size_t lead = i; lead <= d1; ++lead)
    {
        // no separator: digits [lead..) must be non-empty
        size_t k = digits(lead);
        if (k > lead && tail(k)) return true;
        // one arbitrary separator character
        if (lead < n)
        {
            k = digits(lead + 1);
            if (k > lead + 1 && tail(k)) return true;
        }
    }
    return false;
}

bool ExString::strToInt(const std::string &str, int &val)
{
    if (!isNumber(str)) return false;
    val = std::atoi(str.c_str());
    return true;
}

bool ExString::strToFloat(const std::string &str, float &val)
{
    if (!isNumber(str)) return false;
    val = static_cast<float>(std::atof(str.c_str()));
    return true;
}

// ---- Activations name table -----------------------------------------------------------------------------
static const std::pair<const char *, ActivationType> kActNames[] = {
    {"logistic", LOGISTIC}, {"swish", SWISH}, {"hardswish", HARD_SWISH}, {"mish", MISH}, {"normalize_channels", NORM_CHAN},
    {"normalize_channels_softmax", NORM_CHAN_SOFTMAX}, {"normalize_channels_softmax_maxval", NORM_CHAN_SOFTMAX_MAXVAL},
    {"loggy", LOGGY}, {"relu", RELU}, {"prelu", PRELU}, {"relu6", RELU6}, {"elu", ELU}, {"selu", SELU}, {"relie", RELIE},
    {"plse", PLSE}, {"hardtan", HARDTAN}, {"lhtan", LHTAN}, {"ramp", RAMP}, {"leaky", LEAKY}, {"tanh", TANH},
    {"softplus", SOFT_PLUS}, {"stair", STAIR}, {"none", NONE}};

ActivationType Activations::getActivation(const std::string &msg)
{
    for (const auto &e : kActNames)
        if (msg == e.first) return e.second;
    return RELU;
}

std::string Activations::getActivationStr(const ActivationType &type)
{
    switch (type)
    {
    case NORM_CHAN: return "nc";
    case NORM_CHAN_SOFTMAX: return "ncs";
    case NORM_CHAN_SOFTMAX_MAXVAL: return "ncsm";
    default: break;
    }
    for (const auto &e : kActNames)
        if (type == e.second) return e.first;
    return "relu";
}

bool Activations::deviceSupported(const ActivationType &t)
{
    return t == NONE || t == RELU || t == RELU6 || t == LEAKY || t == MISH || t == SWISH || t == HARD_SWISH || t == LOGISTIC;
}

// ---- params ownership -------------------------------------------------------------------------------------
static void freeList(std::vector<BaseParams *> &v)
{
    for (BaseParams *p : v) delete p;
    v.clear();
}

ResBlockParams::~ResBlockParams() { freeList(baseParams); }
Res2BlockParams::~Res2BlockParams() { freeList(baseParams); freeList(branchParams); }
AddBlockParams::~AddBlockParams() { for (auto &b : branchParams) freeList(b); }
ConcatBlockParams::~ConcatBlockParams() { for (auto &b : branchParams) freeList(b); }

Parser::Parser() {}
Parser::~Parser() { clearParams(); }

void Parser::clearParams()
{
    freeList(params);
    BaseParams::index = 0;
}

// ---- scanner ----------------------------------------------------------------------------------------------
std::vector<MsnhNode> Parser::scan(const std::string &text)
{
    struct Row { int indent; std::string key, value; int line; };
    std::vector<Row> rows;
    std::istringstream in(text);
    std::string raw;
    int lineNo = 0;
    while (std::getline(in, raw))
    {
        ++lineNo;
        if (lineNo == 1 && raw.size() >= 3 && static_cast<unsigned char>(raw[0]) == 0xEF) raw = raw.substr(3);   // UTF-8 BOM
        const size_t hash = raw.find('#');
        if (hash != std::string::npos) raw.erase(hash);
        while (!raw.empty() && (raw.back() == ' ' || raw.back() == '\t' || raw.back() == '\r')) raw.pop_back();
        if (raw.empty()) continue;
        size_t ind = 0;
        while (ind < raw.size() && raw[ind] == ' ') ++ind;
        if (ind < raw.size() && raw[ind] == '\t') MSNH_THROW("line " + std::to_string(lineNo) + ": tabs are not allowed for indentation");
        const size_t colon = raw.find(':', ind);
        if (colon == std::string::npos) MSNH_THROW("line " + std::to_string(lineNo) + ": expected 'key: value'");
        Row r;
        r.indent = static_cast<int>(ind);
        r.key = ExString::trim(raw.substr(ind, colon - ind));
        r.value = ExString::trim(raw.substr(colon + 1));
        r.line = lineNo;
        rows.push_back(r);
    }
    size_t pos = 0;
    std::function<std::vector<MsnhNode>(int)> build = [&](int indent) {
        std::vector<MsnhNode> out;
        while (pos < rows.size() && rows[pos].indent == indent)
        {
            MsnhNode n;
            n.key = rows[pos].key;
            n.value = rows[pos].value;
            n.line = rows[pos].line;
            ++pos;
            if (n.value.empty())
            {
                n.isBlock = true;
                if (pos < rows.size() && rows[pos].indent > indent) n.children = build(rows[pos].indent);
            }
            out.push_back(std::move(n));
        }
        if (pos < rows.size() && rows[pos].indent > indent)
            MSNH_THROW("line " + std::to_string(rows[pos].line) + ": bad indentation");
        return out;
    };
    std::vector<MsnhNode> top = build(rows.empty() ? 0 : rows[0].indent);
    if (pos != rows.size()) MSNH_THROW("line " + std::to_string(rows[pos].line) + ": bad indentation");
    return top;
}

// ---- scalar helpers ------------------------------------------------------------------------------------------
namespace
{
void toInt(const MsnhNode &n, const char *owner, int &dst)
{
    if (n.isBlock || !ExString::strToInt(n.value, dst))
        MSNH_THROW(std::string("[") + owner + "] " + n.key + " can't convert to int");
}

void toFloat(const MsnhNode &n, const char *owner, float &dst)
{
    if (n.isBlock || !ExString::strToFloat(n.value, dst))
        MSNH_THROW(std::string("[") + owner + "] " + n.key + " can't convert to float");
}

void toActivation(const MsnhNode &n, ActivationType &act, std::vector<float> &params)
{
    std::vector<std::string> parts;
    ExString::split(parts, n.value, ",");
    if (parts.empty()) { act = Activations::getActivation(""); return; }
    act = Activations::getActivation(parts[0]);
    for (size_t i = 1; i < parts.size(); ++i)
    {
        float v = 0.f;
        ExString::strToFloat(parts[i], v);
        params.push_back(v);
    }
}

[[noreturn]] void unsupportedKey(const MsnhNode &n, const char *owner)
{
    MSNH_THROW(n.key + " is not supported in [" + owner + "]");
}

// resolves the X/Y variants of a scalar parameter: unset (<0) falls back to the scalar
void spread(int scalar, int &x, int &y)
{
    if (x < 0) x = scalar;
    if (y < 0) y = scalar;
}

std::vector<int> layerList(const MsnhNode &n, const char *owner, int ownIndex)
{
    std::vector<std::string> parts;
    ExString::split(parts, n.value, ",");
    std::vector<int> out;
    for (const std::string &p : parts)
    {
        int v = 0;
        if (!ExString::strToInt(p, v)) MSNH_THROW(std::string("[") + owner + "] layers can't convert to int");
        if (v < 0) v = v + ownIndex - 1;          // relative to this layer (src/io/MsnhParser.cpp:2162-2165)
        out.push_back(v);
    }
    return out;
}
} // namespace

// ---- node -> params ---------------------------------------------------------------------------------------------
void Parser::parseSubNodes(const std::vector<MsnhNode> &nodes, const char *owner, std::vector<BaseParams *> &out,
                           const NetConfigParams &cfg, bool allowEmpty)
{
    for (const MsnhNode &n : nodes)
    {
        if (n.key == "size" || n.key == "activation") continue;
        const bool known = n.key == "conv" || n.key == "maxpool" || n.key == "localavgpool" || n.key == "connect" ||
                           n.key == "batchnorm" || (allowEmpty && n.key == "empty");
        if (!known) MSNH_THROW(n.key + " is not supported by [" + owner + "]");
        out.push_back(parseNode(n, false, cfg));
    }
}

static const std::pair<const char *, VariableOpParams::VarOpType> kVarOps[] = {
    {"add", VariableOpParams::VAR_OP_ADD}, {"sub", VariableOpParams::VAR_OP_SUB}, {"subInv", VariableOpParams::VAR_OP_SUB_INV},
    {"mul", VariableOpParams::VAR_OP_MUL}, {"div", VariableOpParams::VAR_OP_DIV}, {"divInv", VariableOpParams::VAR_OP_DIV_INV},
    {"addConst", VariableOpParams::VAR_OP_ADD_CONST}, {"subConst", VariableOpParams::VAR_OP_SUB_CONST},
    {"subConstInv", VariableOpParams::VAR_OP_SUB_CONST_INV}, {"mulConst", VariableOpParams::VAR_OP_MUL_CONST},
    {"divConst", VariableOpParams::VAR_OP_DIV_CONST}, {"divConstInv", VariableOpParams::VAR_OP_DIV_CONST_INV},
    {"abs", VariableOpParams::VAR_OP_ABS}, {"acos", VariableOpParams::VAR_OP_ACOS}, {"asin", VariableOpParams::VAR_OP_ASIN},
    {"atan", VariableOpParams::VAR_OP_ATAN}, {"cos", VariableOpParams::VAR_OP_COS}, {"cosh", VariableOpParams::VAR_OP_COSH},
    {"sin", VariableOpParams::VAR_OP_SIN}, {"sinh", VariableOpParams::VAR_OP_SINH}, {"tan", VariableOpParams::VAR_OP_TAN},
    {"tanh", VariableOpParams::VAR_OP_TANH}, {"exp", VariableOpParams::VAR_OP_EXP}, {"pow", VariableOpParams::VAR_OP_POW},
    {"log", VariableOpParams::VAR_OP_LOG}, {"log10", VariableOpParams::VAR_OP_LOG10}, {"sqrt", VariableOpParams::VAR_OP_SQRT}};

// src/io/MsnhParser.cpp:2278-2392
VariableOpParams::VarOpType VariableOpParams::getVarOpTypeFromStr(const std::string &s)
{
    for (const auto &e : kVarOps)
        if (s == e.first) return e.second;
    MSNH_THROW("[varop] var op no supported : " + s);
}

std::string VariableOpParams::getStrFromVarOpType(const VarOpType &t)
{
    for (const auto &e : kVarOps)
        if (t == e.second) return e.first;
    return "unknown";
}

BaseParams *Parser::parseNode(const MsnhNode &node, bool top, const NetConfigParams &cfg)
{
    const std::string &k = node.key;
    if (k != "empty" && k != "globalavgpool" && !node.isBlock) MSNH_THROW("[" + k + "] content error");

    if (k == "conv")
    {
        std::unique_ptr<ConvParams> p(new ConvParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "batchNorm") toInt(n, "conv", p->batchNorm);
            else if (n.key == "filters") toInt(n, "conv", p->filters);
            else if (n.key == "groups") toInt(n, "conv", p->groups);
            else if (n.key == "kSize") toInt(n, "conv", p->kSize);
            else if (n.key == "kSizeX") toInt(n, "conv", p->kSizeX);
            else if (n.key == "kSizeY") toInt(n, "conv", p->kSizeY);
            else if (n.key == "stride") toInt(n, "conv", p->stride);
            else if (n.key == "strideX") toInt(n, "conv", p->strideX);
            else if (n.key == "strideY") toInt(n, "conv", p->strideY);
            else if (n.key == "dilation") toInt(n, "conv", p->dilation);
            else if (n.key == "dilationX") toInt(n, "conv", p->dilationX);
            else if (n.key == "dilationY") toInt(n, "conv", p->dilationY);
            else if (n.key == "padding") toInt(n, "conv", p->padding);
            else if (n.key == "paddingX") toInt(n, "conv", p->paddingX);
            else if (n.key == "paddingY") toInt(n, "conv", p->paddingY);
            else if (n.key == "antialiasing") toInt(n, "conv", p->antialiasing);
            else if (n.key == "useBias") toInt(n, "conv", p->useBias);
            else if (n.key == "eps") toFloat(n, "conv", p->bnEps);
            else if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else unsupportedKey(n, "conv");
        }
        spread(p->stride, p->strideX, p->strideY);
        spread(p->kSize, p->kSizeX, p->kSizeY);
        spread(p->padding, p->paddingX, p->paddingY);
        spread(p->dilation, p->dilationX, p->dilationY);
        if (p->kSizeX == 1 && p->dilationX > 1) p->dilationX = 1;
        if (p->kSizeY == 1 && p->dilationY > 1) p->dilationY = 1;
        return p.release();
    }
    if (k == "deconv")
    {
        std::unique_ptr<DeConvParams> p(new DeConvParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "filters") toInt(n, "deconv", p->filters);
            else if (n.key == "kSize") toInt(n, "deconv", p->kSize);
            else if (n.key == "kSizeX") toInt(n, "deconv", p->kSizeX);
            else if (n.key == "kSizeY") toInt(n, "deconv", p->kSizeY);
            else if (n.key == "stride") toInt(n, "deconv", p->stride);
            else if (n.key == "strideX") toInt(n, "deconv", p->strideX);
            else if (n.key == "strideY") toInt(n, "deconv", p->strideY);
            else if (n.key == "padding") toInt(n, "deconv", p->padding);
            else if (n.key == "paddingX") toInt(n, "deconv", p->paddingX);
            else if (n.key == "paddingY") toInt(n, "deconv", p->paddingY);
            else if (n.key == "useBias") toInt(n, "deconv", p->useBias);
            else if (n.key == "groups") toInt(n, "deconv", p->groups);
            else if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else unsupportedKey(n, "deconv");
        }
        spread(p->stride, p->strideX, p->strideY);
        spread(p->kSize, p->kSizeX, p->kSizeY);
        spread(p->padding, p->paddingX, p->paddingY);
        return p.release();
    }
    if (k == "batchnorm")
    {
        std::unique_ptr<BatchNormParams> p(new BatchNormParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else if (n.key == "eps") toFloat(n, "batchnorm", p->eps);
            else unsupportedKey(n, "batchnorm");
        }
        return p.release();
    }
    if (k == "maxpool")
    {
        std::unique_ptr<MaxPoolParams> p(new MaxPoolParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "kSize") toInt(n, "maxpool", p->kSize);
            else if (n.key == "kSizeX") toInt(n, "maxpool", p->kSizeX);
            else if (n.key == "kSizeY") toInt(n, "maxpool", p->kSizeY);
            else if (n.key == "stride") toInt(n, "maxpool", p->stride);
            else if (n.key == "strideX") toInt(n, "maxpool", p->strideX);
            else if (n.key == "strideY") toInt(n, "maxpool", p->strideY);
            else if (n.key == "padding") toInt(n, "maxpool", p->padding);
            else if (n.key == "paddingX") toInt(n, "maxpool", p->paddingX);
            else if (n.key == "paddingY") toInt(n, "maxpool", p->paddingY);
            else if (n.key == "maxPoolDepth") toInt(n, "maxpool", p->maxPoolDepth);
            else if (n.key == "outChannels") toInt(n, "maxpool", p->outChannels);
            else if (n.key == "ceilMode") toInt(n, "maxpool", p->ceilMode);
            else if (n.key == "global") toInt(n, "maxpool", p->global);
            else unsupportedKey(n, "maxpool");
        }
        spread(p->stride, p->strideX, p->strideY);
        spread(p->kSize, p->kSizeX, p->kSizeY);
        spread(p->padding, p->paddingX, p->paddingY);
        return p.release();
    }
    if (k == "localavgpool")
    {
        std::unique_ptr<LocalAvgPoolParams> p(new LocalAvgPoolParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "kSize") toInt(n, "localavgpool", p->kSize);
            else if (n.key == "kSizeX") toInt(n, "localavgpool", p->kSizeX);
            else if (n.key == "kSizeY") toInt(n, "localavgpool", p->kSizeY);
            else if (n.key == "stride") toInt(n, "localavgpool", p->stride);
            else if (n.key == "strideX") toInt(n, "localavgpool", p->strideX);
            else if (n.key == "strideY") toInt(n, "localavgpool", p->strideY);
            else if (n.key == "padding") toInt(n, "localavgpool", p->padding);
            else if (n.key == "paddingX") toInt(n, "localavgpool", p->paddingX);
            else if (n.key == "paddingY") toInt(n, "localavgpool", p->paddingY);
            else if (n.key == "ceilMode") toInt(n, "localavgpool", p->ceilMode);
            else if (n.key == "global") toInt(n, "localavgpool", p->global);
            else unsupportedKey(n, "localavgpool");
        }
        spread(p->stride, p->strideX, p->strideY);
        spread(p->kSize, p->kSizeX, p->kSizeY);
        spread(p->padding, p->paddingX, p->paddingY);
        return p.release();
    }
    if (k == "connect")
    {
        std::unique_ptr<ConnectParams> p(new ConnectParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "output") toInt(n, "connect", p->output);
            else if (n.key == "batchNorm") toInt(n, "connect", p->batchNorm);
            else if (n.key == "useBias") toInt(n, "connect", p->useBias);
            else if (n.key == "bnEps") toFloat(n, "connect", p->bnEps);
            else if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else unsupportedKey(n, "connect");
        }
        return p.release();
    }
    if (k == "empty")
    {
        return new EmptyParams(top);
    }
    if (k == "route")
    {
        std::unique_ptr<RouteParams> p(new RouteParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "layers") p->layerIndexes = layerList(n, "route", BaseParams::index);
            else if (n.key == "groups") toInt(n, "route", p->groups);
            else if (n.key == "groupsId") toInt(n, "route", p->groupsId);
            else if (n.key == "addModel") toInt(n, "route", p->addModel);
            else if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else unsupportedKey(n, "route");
        }
        return p.release();
    }
    if (k == "globalavgpool") return new GlobalAvgPoolParams(top);
    if (k == "softmax")
    {
        std::unique_ptr<SoftMaxParams> p(new SoftMaxParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "groups") toInt(n, "softmax", p->groups);
            else if (n.key == "temperature") toFloat(n, "softmax", p->temperature);
            else unsupportedKey(n, "softmax");
        }
        return p.release();
    }
    if (k == "act")
    {
        std::unique_ptr<ActivationParams> p(new ActivationParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "activation") toActivation(n, p->activation, p->actParams);
            else unsupportedKey(n, "act");
        }
        return p.release();
    }
    if (k == "padding")
    {
        std::unique_ptr<PaddingParams> p(new PaddingParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "top") toInt(n, "padding", p->top);
            else if (n.key == "down") toInt(n, "padding", p->down);
            else if (n.key == "left") toInt(n, "padding", p->left);
            else if (n.key == "right") toInt(n, "padding", p->right);
            else if (n.key == "paddingVal") toFloat(n, "padding", p->paddingVal);
            else unsupportedKey(n, "padding");
        }
        return p.release();
    }
    if (k == "slice")
    {
        std::unique_ptr<SliceParams> p(new SliceParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "start0") toInt(n, "slice", p->start0);
            else if (n.key == "step0") toInt(n, "slice", p->step0);
            else if (n.key == "start1") toInt(n, "slice", p->start1);
            else if (n.key == "step1") toInt(n, "slice", p->step1);
            else if (n.key == "start2") toInt(n, "slice", p->start2);
            else if (n.key == "step2") toInt(n, "slice", p->step2);
            else unsupportedKey(n, "slice");
        }
        return p.release();
    }
    if (k == "varop")
    {
        std::unique_ptr<VariableOpParams> p(new VariableOpParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "layers") p->layerIndexes = layerList(n, "varop", BaseParams::index);
            else if (n.key == "type") p->varOpType = VariableOpParams::getVarOpTypeFromStr(n.value);
            else if (n.key == "constVal") toFloat(n, "varop", p->constVal);
            else unsupportedKey(n, "varop");
        }
        return p.release();
    }
    if (k == "upsample")
    {
        std::unique_ptr<UpSampleParams> p(new UpSampleParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "stride") toInt(n, "unsample", p->stride);
            else if (n.key == "strideX") toInt(n, "unsample", p->strideX);
            else if (n.key == "strideY") toInt(n, "unsample", p->strideY);
            else if (n.key == "scale") toFloat(n, "unsample", p->scale);
            else if (n.key == "scaleX") toFloat(n, "unsample", p->scaleX);
            else if (n.key == "scaleY") toFloat(n, "unsample", p->scaleY);
            else if (n.key == "alignCorners") toInt(n, "unsample", p->alignCorners);
            else if (n.key == "type")
            {
                if (n.value == "nearest") p->upsampleType = UpSampleParams::NEAREST;
                else if (n.value == "bilinear") p->upsampleType = UpSampleParams::BILINEAR;
                else MSNH_THROW("[unsample] type " + n.value + " is not supported");
            }
            else unsupportedKey(n, "unsample");
        }
        spread(p->stride, p->strideX, p->strideY);
        if (p->scaleX < 0) p->scaleX = p->scale;
        if (p->scaleY < 0) p->scaleY = p->scale;
        return p.release();
    }
    if (k == "yolo")
    {
        std::unique_ptr<YoloParams> p(new YoloParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "anchors")
            {
                std::vector<std::string> parts;
                ExString::split(parts, n.value, ",");
                if (parts.size() != 6) MSNH_THROW("[yolo] anchor num should be 6");
                for (const std::string &s : parts)
                {
                    float v = 0.f;
                    if (!ExString::strToFloat(ExString::trim(s), v)) MSNH_THROW("[yolo] anchors can't convert to float");
                    p->anchors.push_back(v);
                }
            }
            else if (n.key == "classNum") toInt(n, "yolo", p->classNum);
            else if (n.key == "yoloType") p->yoloType = getYoloTypeFromStr(n.value);
            else unsupportedKey(n, "yolo");
        }
        p->orgHeight = cfg.height;
        p->orgWidth = cfg.width;
        return p.release();
    }
    if (k == "yoloout")
    {
        std::unique_ptr<YoloOutParams> p(new YoloOutParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "layers") p->layerIndexes = layerList(n, "yoloout", BaseParams::index);
            else if (n.key == "confThresh") toFloat(n, "yoloout", p->confThresh);
            else if (n.key == "nmsThresh") toFloat(n, "yoloout", p->nmsThresh);
            else if (n.key == "useSoftNms") toInt(n, "yoloout", p->useSoftNms);
            else if (n.key == "yoloType") p->yoloType = getYoloTypeFromStr(n.value);
            else unsupportedKey(n, "yoloout");
        }
        p->orgHeight = cfg.height;
        p->orgWidth = cfg.width;
        return p.release();
    }
    if (k == "resblock")
    {
        std::unique_ptr<ResBlockParams> p(new ResBlockParams(top));
        parseSubNodes(node.children, "ResBlockLayer", p->baseParams, cfg, false);
        return p.release();
    }
    if (k == "res2block")
    {
        std::unique_ptr<Res2BlockParams> p(new Res2BlockParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "size" || n.key == "activation") continue;
            if (n.key == "base") parseSubNodes(n.children, "Res2BlockLayer", p->baseParams, cfg, false);
            else if (n.key == "branch") parseSubNodes(n.children, "Res2BlockLayer", p->branchParams, cfg, false);
            else unsupportedKey(n, "res2block");
        }
        return p.release();
    }
    if (k == "addblock")
    {
        std::unique_ptr<AddBlockParams> p(new AddBlockParams(top));
        for (const MsnhNode &n : node.children)
        {
            if (n.key == "size" || n.key == "activation") continue;
            if (n.key != "branch") unsupportedKey(n, "addblock");
            p->branchParams.emplace_back();
            parseSubNodes(n.children, "AddBlockLayer", p->branchParams.back(), cfg, true);
        }
        return p.release();
    }
    if (k == "concatblock")
    {
        std::unique_ptr<ConcatBlockParams> p(new ConcatBlockParams(top));
        for (const MsnhNode &n : node.children)
        {
            // The reference appends a branch for every key of the block, `size` and `activation` included
            // (src/io/MsnhParser.cpp:1972-2054), which makes such files unusable there; they are refused here.
            if (n.key != "branch") MSNH_THROW(n.key + " is not supported in [concatblock]: only branch nodes are allowed");
            p->branchParams.emplace_back();
            parseSubNodes(n.children, "ConcatBlockLayer", p->branchParams.back(), cfg, true);
        }
        return p.release();
    }
    MSNH_THROW("[" + k + "] layer type is outside the convolutional path this build implements");
}

void Parser::readCfg(const std::string &path)
{
    clearParams();
    std::ifstream f(path, std::ios::binary);
    if (!f.is_open()) MSNH_THROW("msnhnet file: " + path + " open failed");
    std::stringstream ss;
    ss << f.rdbuf();
    const std::vector<MsnhNode> nodes = scan(ss.str());
    if (nodes.empty() || nodes[0].key != "config") MSNH_THROW("first node must be [config]");
    if (!nodes[0].isBlock) MSNH_THROW("[config] content error");

    NetConfigParams *cfg = new NetConfigParams(false);
    params.push_back(cfg);
    for (const MsnhNode &n : nodes[0].children)
    {
        if (n.key == "batch") toInt(n, "config", cfg->batch);
        else if (n.key == "width") toInt(n, "config", cfg->width);
        else if (n.key == "height") toInt(n, "config", cfg->height);
        else if (n.key == "channels") toInt(n, "config", cfg->channels);
        else unsupportedKey(n, "config");
    }

    for (size_t i = 1; i < nodes.size(); ++i)
    {
        const MsnhNode &n = nodes[i];
        int copies = 1;
        ActivationType act = ActivationType::NONE;
        std::vector<float> actParams;
        const bool sized = n.key == "resblock" || n.key == "res2block" || n.key == "addblock";
        if (sized || n.key == "concatblock")
        {
            if (!n.isBlock) MSNH_THROW("[" + n.key + "] content error");
            for (const MsnhNode &c : n.children)
            {
                if (sized && c.key == "size") toInt(c, n.key.c_str(), copies);
                if (sized && c.key == "activation") toActivation(c, act, actParams);
            }
        }
        for (int r = 0; r < copies; ++r)
        {
            BaseParams *p = parseNode(n, true, *cfg);
            // the block's activation parameters are dropped for resblock, kept for the other blocks
            // (src/io/MsnhParser.cpp:413, 470, 527)
            if (n.key == "resblock") static_cast<ResBlockParams *>(p)->activation = act;
            else if (n.key == "res2block") { static_cast<Res2BlockParams *>(p)->activation = act; static_cast<Res2BlockParams *>(p)->actParams = actParams; }
            else if (n.key == "addblock") { static_cast<AddBlockParams *>(p)->activation = act; static_cast<AddBlockParams *>(p)->actParams = actParams; }
            params.push_back(p);
        }
    }
}

void Parser::readMsnhBin(const std::string &path)
{
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f.is_open()) MSNH_THROW("msnhbin file: " + path + " open failed");
    const std::streamoff bytes = f.tellg();
    if (bytes % 4 != 0) MSNH_THROW("msnhbin file size error");
    msnhF32Weights.resize(static_cast<size_t>(bytes / 4));
    f.seekg(0);
    if (bytes > 0) f.read(reinterpret_cast<char *>(msnhF32Weights.data()), bytes);       // little-endian float32, no header
    if (!f) MSNH_THROW("msnhbin file: " + path + " read failed");
}
}
