// Wall-clock helper (milliseconds), as used for the per-layer time table.
#pragma once
#include <chrono>

namespace Msnhnet
{
class TimeUtil
{
public:
    static std::chrono::high_resolution_clock::time_point startRecord() { return std::chrono::high_resolution_clock::now(); }
    static float getElapsedTime(const std::chrono::high_resolution_clock::time_point &st)
    {
        return std::chrono::duration<float, std::milli>(std::chrono::high_resolution_clock::now() - st).count();
    }
};
}
