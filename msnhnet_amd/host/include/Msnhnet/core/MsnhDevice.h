// Thin C++ wrappers over the kernel library's C ABI (include/msnh_hip.h): error translation into
// Msnhnet::Exception (the reference exits the process on device errors, src/config/MsnhnetCuda.cpp:18-56)
// and RAII ownership of device / pinned-host buffers.  The host library contains no HIP code of its own.
#pragma once
#include <string>
#include <vector>
#include "msnh_hip.h"
#include "Msnhnet/utils/MsnhException.h"

namespace Msnhnet
{
#define MSNH_DEV(call)                                                                                          \
    do {                                                                                                        \
        if ((call) != 0) throw ::Msnhnet::Exception(1, std::string("device: ") + msnh_hip_last_error(), __FILE__, __LINE__, __FUNCTION__); \
    } while (0)

class Device
{
public:
    // Selects device 0 once per process; throws if no GPU is usable.  There is no CPU fallback.
    static void ensureInit();
    static bool initialised();
};

class DeviceBuffer
{
public:
    DeviceBuffer() {}
    explicit DeviceBuffer(size_t bytes) { alloc(bytes); }
    ~DeviceBuffer() { release(); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : _ptr(o._ptr), _bytes(o._bytes), _owned(o._owned) { o._ptr = nullptr; o._bytes = 0; o._owned = true; }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept
    {
        if (this != &o) { release(); _ptr = o._ptr; _bytes = o._bytes; _owned = o._owned; o._ptr = nullptr; o._bytes = 0; o._owned = true; }
        return *this;
    }
    void alloc(size_t bytes)
    {
        release();
        Device::ensureInit();
        MSNH_DEV(msnh_hip_malloc(&_ptr, bytes));
        _bytes = bytes;
    }
    void release()
    {
        if (_ptr && _owned) msnh_hip_free(_ptr);
        _ptr = nullptr;
        _bytes = 0;
        _owned = true;
    }
    // A view of another buffer's memory: nothing is freed when this object goes away; the owner must outlive it.
    void aliasOf(const DeviceBuffer &o)
    {
        release();
        _ptr = o._ptr;
        _bytes = o._bytes;
        _owned = false;
    }
    void upload(const void *host, size_t bytes, msnh_stream_t s = nullptr)
    {
        if (bytes > _bytes) alloc(bytes);
        MSNH_DEV(msnh_hip_memcpy_h2d(_ptr, host, bytes, s));
        MSNH_DEV(msnh_hip_stream_sync(s));
    }
    void *ptr() const { return _ptr; }
    size_t bytes() const { return _bytes; }
    template <typename T> T *as() const { return static_cast<T *>(_ptr); }

private:
    void  *_ptr = nullptr;
    size_t _bytes = 0;
    bool   _owned = true;
};

class PinnedBuffer
{
public:
    PinnedBuffer() {}
    ~PinnedBuffer() { release(); }
    PinnedBuffer(const PinnedBuffer &) = delete;
    PinnedBuffer &operator=(const PinnedBuffer &) = delete;
    void reserve(size_t bytes)
    {
        if (bytes <= _bytes) return;
        release();
        Device::ensureInit();
        MSNH_DEV(msnh_hip_host_alloc(&_ptr, bytes));
        _bytes = bytes;
    }
    void release()
    {
        if (_ptr) msnh_hip_host_free(_ptr);
        _ptr = nullptr;
        _bytes = 0;
    }
    void *ptr() const { return _ptr; }
    template <typename T> T *as() const { return static_cast<T *>(_ptr); }
    size_t bytes() const { return _bytes; }

private:
    void  *_ptr = nullptr;
    size_t _bytes = 0;
};
}
