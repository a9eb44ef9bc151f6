// Msnhnet::Exception -- the one exception type thrown by the host side (same constructor arguments and
// getters as the reference's include/Msnhnet/utils/MsnhException.h:10-61).
#pragma once
#include <exception>
#include <string>
#include "Msnhnet/config/MsnhnetCfg.h"

namespace Msnhnet
{
class MsnhNet_API Exception : public std::exception
{
public:
    Exception() : _what("error") {}
    Exception(int errCode, std::string err, std::string errFile, int errLine, std::string errFun)
        : _what(std::move(err)), _file(std::move(errFile)), _fun(std::move(errFun)), _code(errCode), _line(errLine) {}

    const char *what() const noexcept override { return _what.c_str(); }
    std::string getErrFile() const { return _file; }
    std::string getErrFun() const { return _fun; }
    int getErrLine() const { return _line; }
    int getErrCode() const { return _code; }

private:
    std::string _what, _file, _fun;
    int _code = 0, _line = 0;
};
}

#define MSNH_THROW(msg) throw ::Msnhnet::Exception(1, (msg), __FILE__, __LINE__, __FUNCTION__)
