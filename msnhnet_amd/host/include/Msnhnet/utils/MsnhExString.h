// String helpers used by the `.msnhnet` reader.
#pragma once
#include <string>
#include <vector>
#include "Msnhnet/config/MsnhnetCfg.h"

namespace Msnhnet
{
class MsnhNet_API ExString
{
public:
    // Splits on any character of `cutset`; empty tokens vanish (strtok semantics, src/utils/MsnhExString.cpp:5-22).
    static void split(std::vector<std::string> &result, const std::string &str, const std::string &cutset);
    static std::string trim(const std::string &str);
    // Accept only strings matching [-+]?[0-9]*.?[0-9]+([eE][-+]?[0-9]+)? (src/utils/MsnhExString.cpp:126-144).
    static bool isNumber(const std::string &str);
    static bool strToInt(const std::string &str, int &val);
    static bool strToFloat(const std::string &str, float &val);
};
}
