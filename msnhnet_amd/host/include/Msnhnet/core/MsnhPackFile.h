// The packed device-side constants of one plan, kept beside the weights file ("<weights>.f16.pack" / ".f32.pack") so that the next load of
// the same graph with the same weights neither runs the float32 calibration pass nor re-packs the kernels.
//
// The reference keeps nothing between loads: every start reads the float32 weights (src/net/MsnhNetBuilder.cpp:624-663) and, in its
// float16 mode, converts them on the device again (src/layers/MsnhConvolutionalLayer.cpp:loadAllWeigths).
//
// File: one text line (format version, packing layout version of the kernel library, number of tile configurations, Winograd preference,
// dtype), then binary little-endian: hash of the weights file, hash of the plan's structure, tensor count, the calibrated absolute maximum
// of every tensor, then one record per packed blob { op index, algorithm, byte count, hash of the bytes, bytes padded to 8 } and a closing record that holds
// the number of blobs.  A file whose line or hashes differ, that is cut short, that holds a blob whose bytes no longer hash to the recorded
// value, or that lacks a blob the plan asks for is ignored and rewritten.
#pragma once
#include <cstdint>
#include <cstdio>
#include <memory>
#include <string>
#include <vector>

namespace Msnhnet
{
class PackFile
{
public:
    ~PackFile();
    static std::string headerLine(int dtype, bool preferWinograd);
    static uint64_t hash(const void *data, size_t bytes, uint64_t seed = 0);

    // reading: false if the file is absent or does not belong to this (library, weights, plan)
    bool open(const std::string &path, const std::string &header, uint64_t weightsHash, uint64_t graphHash, size_t nTensors);
    const std::vector<float> &amax() const { return _amax; }
    // the blob recorded for launch `op` under `algo`, nullptr (and the file counts as stale) if there is none of exactly `bytes` bytes
    const unsigned char *blob(uint32_t op, uint32_t algo, size_t bytes);
    bool stale() const { return _stale; }
    size_t blobsServed() const { return _served; }

    // writing: into "<path>.tmp.<pid>.<n>", renamed over `path` by commit()
    bool create(const std::string &path, const std::string &header, uint64_t weightsHash, uint64_t graphHash, const std::vector<float> &amax);
    void add(uint32_t op, uint32_t algo, const void *data, size_t bytes);
    bool commit();

private:
    struct Entry { uint32_t op, algo; size_t offset, bytes; };
    std::unique_ptr<unsigned char[]> _file;
    std::vector<Entry> _entries;
    std::vector<float> _amax;
    bool _stale = false;
    size_t _served = 0;
    std::FILE *_out = nullptr;
    std::string _path, _tmp;
    uint32_t _written = 0;
    bool _failed = false;
};
}
