// `.msnhnet` graph reader and `.msnhbin` weight reader.
//
// A `.msnhnet` file is one YAML mapping whose keys repeat and whose document order is the layer order
// (src/io/MsnhParser.cpp:140-682).  That is not valid YAML for a general loader, so this reader is a small
// indentation-based scanner for exactly that subset: `key: value` scalars, nested blocks, `#` comments.
// The *Params classes keep the reference's names and fields (include/Msnhnet/io/MsnhParser.h:16-565) for the
// node types of the convolutional path; node types outside it are rejected with a clear message.
#pragma once
#include <cfloat>
#include <memory>
#include <string>
#include <vector>
#include "Msnhnet/config/MsnhnetCfg.h"
#include "Msnhnet/layers/MsnhActivations.h"
#include "Msnhnet/layers/MsnhYoloDef.h"
#include "Msnhnet/utils/MsnhExString.h"

namespace Msnhnet
{
class MsnhNet_API BaseParams
{
public:
    explicit BaseParams(bool incIndex) { if (incIndex) index++; }
    virtual ~BaseParams() {}
    LayerType type = LayerType::CONFIG;
    static int index;            // 1 + index of the top-level layer being parsed (negative route refs use it)
};

class MsnhNet_API NetConfigParams : public BaseParams
{
public:
    explicit NetConfigParams(bool inc) : BaseParams(inc) { type = LayerType::CONFIG; }
    int batch = 1, width = 0, height = 0, channels = 0;
};

class MsnhNet_API EmptyParams : public BaseParams
{
public:
    explicit EmptyParams(bool inc) : BaseParams(inc) { type = LayerType::EMPTY; }
};

class MsnhNet_API ConvParams : public BaseParams
{
public:
    explicit ConvParams(bool inc) : BaseParams(inc) { type = LayerType::CONVOLUTIONAL; }
    int batchNorm = 0, filters = 1, groups = 1;
    int kSize = 1, kSizeX = -1, kSizeY = -1;
    int stride = 1, strideX = -1, strideY = -1;
    int antialiasing = 0;
    int padding = 0, paddingX = -1, paddingY = -1;
    int dilation = 1, dilationX = -1, dilationY = -1;
    int useBias = 1;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
    float bnEps = 0.00001f;
};

class MsnhNet_API DeConvParams : public BaseParams
{
public:
    explicit DeConvParams(bool inc) : BaseParams(inc) { type = LayerType::DECONVOLUTIONAL; }
    int filters = 1, groups = 1, useBias = 1;
    int kSize = 1, kSizeX = -1, kSizeY = -1;
    int stride = 1, strideX = -1, strideY = -1;
    int padding = 0, paddingX = -1, paddingY = -1;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API MaxPoolParams : public BaseParams
{
public:
    explicit MaxPoolParams(bool inc) : BaseParams(inc) { type = LayerType::MAXPOOL; }
    int kSize = 1, kSizeX = -1, kSizeY = -1;
    int stride = 1, strideX = -1, strideY = -1;
    int padding = 0, paddingX = -1, paddingY = -1;
    int maxPoolDepth = 0, outChannels = 1, ceilMode = 0, global = 0;
};

class MsnhNet_API LocalAvgPoolParams : public BaseParams
{
public:
    explicit LocalAvgPoolParams(bool inc) : BaseParams(inc) { type = LayerType::LOCAL_AVGPOOL; }
    int kSize = 1, kSizeX = -1, kSizeY = -1;
    int stride = 1, strideX = -1, strideY = -1;
    int padding = 0, paddingX = -1, paddingY = -1;
    int ceilMode = 0, global = 0;
};

class MsnhNet_API ConnectParams : public BaseParams
{
public:
    explicit ConnectParams(bool inc) : BaseParams(inc) { type = LayerType::CONNECTED; }
    int output = 0, batchNorm = 0, useBias = 1;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
    float bnEps = 0.00001f;
};

class MsnhNet_API BatchNormParams : public BaseParams
{
public:
    explicit BatchNormParams(bool inc) : BaseParams(inc) { type = LayerType::BATCHNORM; }
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
    float eps = 0.00001f;
};

// Blocks own their sub-node params.
class MsnhNet_API ResBlockParams : public BaseParams
{
public:
    explicit ResBlockParams(bool inc) : BaseParams(inc) { type = LayerType::RES_BLOCK; }
    ~ResBlockParams() override;
    std::vector<BaseParams *> baseParams;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API Res2BlockParams : public BaseParams
{
public:
    explicit Res2BlockParams(bool inc) : BaseParams(inc) { type = LayerType::RES_2_BLOCK; }
    ~Res2BlockParams() override;
    std::vector<BaseParams *> baseParams, branchParams;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API AddBlockParams : public BaseParams
{
public:
    explicit AddBlockParams(bool inc) : BaseParams(inc) { type = LayerType::ADD_BLOCK; }
    ~AddBlockParams() override;
    std::vector<std::vector<BaseParams *>> branchParams;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API ConcatBlockParams : public BaseParams
{
public:
    explicit ConcatBlockParams(bool inc) : BaseParams(inc) { type = LayerType::CONCAT_BLOCK; }
    ~ConcatBlockParams() override;
    std::vector<std::vector<BaseParams *>> branchParams;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API RouteParams : public BaseParams
{
public:
    explicit RouteParams(bool inc) : BaseParams(inc) { type = LayerType::ROUTE; }
    std::vector<int> layerIndexes;
    int groups = 1, groupsId = 0, addModel = 0;
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API GlobalAvgPoolParams : public BaseParams
{
public:
    explicit GlobalAvgPoolParams(bool inc) : BaseParams(inc) { type = LayerType::GLOBAL_AVGPOOL; }
};

class MsnhNet_API SoftMaxParams : public BaseParams
{
public:
    explicit SoftMaxParams(bool inc) : BaseParams(inc) { type = LayerType::SOFTMAX; }
    int groups = 1;
    float temperature = 1;
};

class MsnhNet_API ActivationParams : public BaseParams
{
public:
    explicit ActivationParams(bool inc) : BaseParams(inc) { type = LayerType::ACTIVE; }
    ActivationType activation = ActivationType::NONE;
    std::vector<float> actParams;
};

class MsnhNet_API PaddingParams : public BaseParams
{
public:
    explicit PaddingParams(bool inc) : BaseParams(inc) { type = LayerType::PADDING; }
    int top = 0, down = 0, left = 0, right = 0;
    float paddingVal = 0;
};

class MsnhNet_API SliceParams : public BaseParams
{
public:
    explicit SliceParams(bool inc) : BaseParams(inc) { type = LayerType::SLICE; }
    int start0 = 0, step0 = 1, start1 = 0, step1 = 1, start2 = 0, step2 = 1;
};

class MsnhNet_API VariableOpParams : public BaseParams
{
public:
    enum VarOpType
    {
        VAR_OP_ADD = 0, VAR_OP_SUB, VAR_OP_SUB_INV, VAR_OP_MUL, VAR_OP_DIV, VAR_OP_DIV_INV,
        VAR_OP_ADD_CONST, VAR_OP_SUB_CONST, VAR_OP_SUB_CONST_INV, VAR_OP_MUL_CONST, VAR_OP_DIV_CONST, VAR_OP_DIV_CONST_INV,
        VAR_OP_ABS, VAR_OP_ACOS, VAR_OP_ASIN, VAR_OP_ATAN, VAR_OP_COS, VAR_OP_COSH, VAR_OP_SIN, VAR_OP_SINH, VAR_OP_TAN, VAR_OP_TANH,
        VAR_OP_EXP, VAR_OP_POW, VAR_OP_LOG, VAR_OP_LOG10, VAR_OP_SQRT
    };
    explicit VariableOpParams(bool inc) : BaseParams(inc) { type = LayerType::VARIABLE_OP; }
    std::vector<int> layerIndexes;
    VarOpType varOpType = VAR_OP_ADD;
    float constVal = 0;
    static VarOpType getVarOpTypeFromStr(const std::string &s);
    static std::string getStrFromVarOpType(const VarOpType &t);
};

class MsnhNet_API UpSampleParams : public BaseParams
{
public:
    enum UpsampleType { NEAREST = 0, BILINEAR };
    explicit UpSampleParams(bool inc) : BaseParams(inc) { type = LayerType::UPSAMPLE; }
    int   stride = 1, strideX = -1, strideY = -1;
    float scale = 1.f, scaleX = -1.f, scaleY = -1.f;
    int   alignCorners = 0;
    UpsampleType upsampleType = NEAREST;
};

class MsnhNet_API YoloParams : public BaseParams
{
public:
    explicit YoloParams(bool inc) : BaseParams(inc) { type = LayerType::YOLO; }
    int orgWidth = 0, orgHeight = 0, classNum = 1;
    std::vector<float> anchors;
    YoloType yoloType = YoloType::YoloV3;
};

class MsnhNet_API YoloOutParams : public BaseParams
{
public:
    explicit YoloOutParams(bool inc) : BaseParams(inc) { type = LayerType::YOLO_OUT; }
    std::vector<int> layerIndexes;
    float confThresh = 0, nmsThresh = 0;
    int   useSoftNms = 0;
    int   orgWidth = 0, orgHeight = 0;
    YoloType yoloType = YoloType::YoloV3;
};

// One scanned node of the file: a scalar (`children` empty) or a block.
struct MsnhNode
{
    std::string key, value;
    int line = 0;
    bool isBlock = false;
    std::vector<MsnhNode> children;
};

class MsnhNet_API Parser
{
public:
    Parser();
    ~Parser();

    std::vector<BaseParams *> params;          // params[0] is the NetConfigParams
    std::vector<float> msnhF32Weights;

    void clearParams();
    void readCfg(const std::string &path);     // throws Msnhnet::Exception on any malformed input
    void readMsnhBin(const std::string &path);

    // text -> node tree (exposed for tests)
    static std::vector<MsnhNode> scan(const std::string &text);

private:
    BaseParams *parseNode(const MsnhNode &node, bool topLevel, const NetConfigParams &cfg);
    void parseSubNodes(const std::vector<MsnhNode> &nodes, const char *owner, std::vector<BaseParams *> &out,
                       const NetConfigParams &cfg, bool allowEmpty);
};
}
