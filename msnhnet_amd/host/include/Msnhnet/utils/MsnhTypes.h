// Small value types: Point2I and the box helpers used by the YOLO post-processing.
#pragma once
#include <algorithm>
#include "Msnhnet/config/MsnhnetCfg.h"

namespace Msnhnet
{
struct Point2I
{
    Point2I() {}
    Point2I(int x, int y) : x(x), y(y) {}
    int x = 0;
    int y = 0;
};

class Box
{
public:
    struct XYWHBox
    {
        XYWHBox() {}
        XYWHBox(float x, float y, float w, float h) : x(x), y(y), w(w), h(h) {}
        float x = 0, y = 0, w = 0, h = 0;
    };

    struct X1Y1X2Y2Box
    {
        X1Y1X2Y2Box() {}
        X1Y1X2Y2Box(float x1, float y1, float x2, float y2) : x1(x1), y1(y1), x2(x2), y2(y2) {}
        float x1 = 0, y1 = 0, x2 = 0, y2 = 0;
    };

    static X1Y1X2Y2Box toX1Y1X2Y2Box(const XYWHBox &b)
    {
        return X1Y1X2Y2Box(b.x - b.w / 2.f, b.y - b.h / 2.f, b.x + b.w / 2.f, b.y + b.h / 2.f);
    }

    static XYWHBox toXYWHBox(const X1Y1X2Y2Box &b)
    {
        const float w = b.x2 - b.x1, h = b.y2 - b.y1;
        return XYWHBox(b.x1 + w / 2.f, b.y1 + h / 2.f, w, h);
    }

    // Intersection over union with the reference's inclusive-pixel (+1) convention
    // (include/Msnhnet/utils/MsnhTypes.h:123-140); NaN/inf operands propagate exactly as there.
    static float iou(const XYWHBox &p, const XYWHBox &q)
    {
        const X1Y1X2Y2Box a = toX1Y1X2Y2Box(p), b = toX1Y1X2Y2Box(q);
        const float iw = std::min(a.x2, b.x2) - std::max(a.x1, b.x1) + 1;
        const float ih = std::min(a.y2, b.y2) - std::max(a.y1, b.y1) + 1;
        const float inter = (iw < 0 ? 0 : iw) * (ih < 0 ? 0 : ih);
        const float areaA = (a.x2 - a.x1 + 1) * (a.y2 - a.y1 + 1);
        const float areaB = (b.x2 - b.x1 + 1) * (b.y2 - b.y1 + 1);
        return 1.f * inter / (areaA + areaB - inter);
    }
};
}
