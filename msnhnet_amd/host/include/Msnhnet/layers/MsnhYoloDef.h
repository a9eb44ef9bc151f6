// YOLO value types: YoloBox (one detection), YoloInfo (geometry of one head), YoloType.
// Field names and enum values follow include/Msnhnet/layers/MsnhYoloDef.h:8-110.
#pragma once
#include <string>
#include <vector>
#include "Msnhnet/utils/MsnhException.h"
#include "Msnhnet/utils/MsnhTypes.h"

namespace Msnhnet
{
struct YoloInfo
{
    YoloInfo(int outHeight, int outWidth, int outChannel) : outHeight(outHeight), outWidth(outWidth), outChannel(outChannel) {}
    int outHeight = 0, outWidth = 0, outChannel = 0;
    int getOutputNum() const { return outChannel * outWidth * outHeight; }
};

struct YoloBox
{
    Box::XYWHBox xywhBox;
    float conf = 0;
    float bestClsConf = 0;
    int   bestClsIdx = 0;
    float angle = 0;
    float regAngle = 0;
    std::vector<float> classesVal;      // filled only when NetBuilder::setKeepClassScores(true)
    std::vector<float> angleSplits;
};

enum YoloType { YoloV3 = 30, YoloV3_ANGLE, YoloV3_GAUSSIAN, YoloV4 = 40, YoloV4_ANGLE, YoloV5 = 50, YoloV5_ANGLE };

inline YoloType getYoloTypeFromStr(const std::string &s)
{
    static const std::pair<const char *, YoloType> table[] = {
        {"yolov3", YoloV3}, {"yolov3Angle", YoloV3_ANGLE}, {"yolov3Gaussian", YoloV3_GAUSSIAN}, {"yolov4", YoloV4},
        {"yolov4Angle", YoloV4_ANGLE}, {"yolov5", YoloV5}, {"yolov5Angle", YoloV5_ANGLE}};
    for (const auto &e : table)
        if (s == e.first) return e.second;
    MSNH_THROW(s + " yolo type is not supported!");
}

inline std::string getStrFromYoloType(const YoloType &t)
{
    switch (t)
    {
    case YoloV3: return "yolov3";
    case YoloV3_ANGLE: return "yolov3Angle";
    case YoloV3_GAUSSIAN: return "yolov3Gaussian";
    case YoloV4: return "yolov4";
    case YoloV4_ANGLE: return "yolov4Angle";
    case YoloV5: return "yolov5";
    case YoloV5_ANGLE: return "yolov5Angle";
    }
    MSNH_THROW(std::to_string(static_cast<int>(t)) + " yolo type is not supported!");
}
}
