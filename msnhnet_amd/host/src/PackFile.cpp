// Reader and writer of the packed-constants file of a plan (layout in MsnhPackFile.h).
#include "Msnhnet/core/MsnhPackFile.h"
#include <atomic>
#include <cstring>
#include <unistd.h>
#include "msnh_hip.h"

namespace Msnhnet
{
namespace
{
constexpr int kFormat = 2;
constexpr uint32_t kClosing = 0xFFFFFFFFu;
struct Record { uint32_t op, algo; uint64_t bytes, hash; };          // hash: PackFile::hash of the blob (the closing record: 0)
// two processes (or two NetBuilders of one process) that write the file of the same weights at the same time each use a name of their own
std::string tempName(const std::string &path)
{
    static std::atomic<unsigned> counter{0};
    return path + ".tmp." + std::to_string(static_cast<long long>(getpid())) + "." + std::to_string(counter++);
}
}

PackFile::~PackFile()
{
    if (_out)
    {
        std::fclose(_out);
        std::remove(_tmp.c_str());
    }
}

std::string PackFile::headerLine(int dtype, bool preferWinograd)
{
    return "msnhpack " + std::to_string(kFormat) + " layout " + std::to_string(msnh_hip_conv2d_pack_layout_version()) + " tiles " +
           std::to_string(msnh_hip_conv2d_tile_count()) + " winograd " + std::to_string(preferWinograd ? 1 : 0) + " dtype " + std::to_string(dtype);
}

// 64-bit multiply-xorshift over 8-byte words, four independent lanes (a checksum of a few hundred MB in tens of milliseconds; not
// cryptographic: it guards against a stale file, not against an adversary)
uint64_t PackFile::hash(const void *data, size_t bytes, uint64_t seed)
{
    const unsigned char *p = static_cast<const unsigned char *>(data);
    uint64_t h[4] = {0x9E3779B97F4A7C15ull ^ seed, 0xC2B2AE3D27D4EB4Full + seed, 0x165667B19E3779F9ull ^ (seed << 1), 0x27D4EB2F165667C5ull + bytes};
    const uint64_t m = 0xFF51AFD7ED558CCDull;
    size_t i = 0;
    for (; i + 32 <= bytes; i += 32)
    {
        uint64_t w[4];
        std::memcpy(w, p + i, 32);
        for (int k = 0; k < 4; ++k)
        {
            h[k] = (h[k] ^ w[k]) * m;
            h[k] ^= h[k] >> 29;
        }
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    std::memcpy(tail, p + i, bytes - i);
    uint64_t r = bytes;
    for (int k = 0; k < 4; ++k)
    {
        h[k] = (h[k] ^ tail[k]) * m;
        h[k] ^= h[k] >> 29;
        r = (r ^ h[k]) * 0xC4CEB9FE1A85EC53ull;
        r ^= r >> 32;
    }
    return r;
}

bool PackFile::open(const std::string &path, const std::string &header, uint64_t weightsHash, uint64_t graphHash, size_t nTensors)
{
    std::FILE *f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    bool ok = std::fseek(f, 0, SEEK_END) == 0;
    const long total = ok ? std::ftell(f) : -1;
    ok = ok && total > 0 && std::fseek(f, 0, SEEK_SET) == 0;
    const size_t fixed = header.size() + 1 + 3 * sizeof(uint64_t) + nTensors * sizeof(float);
    ok = ok && static_cast<size_t>(total) >= fixed + sizeof(Record);
    // the line and the hashes first: a file that belongs to something else is not read any further
    std::vector<unsigned char> head(ok ? fixed : 0);
    ok = ok && std::fread(head.data(), 1, fixed, f) == fixed && std::memcmp(head.data(), header.data(), header.size()) == 0 && head[header.size()] == '\n';
    uint64_t three[3] = {0, 0, 0};
    if (ok) std::memcpy(three, head.data() + header.size() + 1, sizeof(three));
    ok = ok && three[0] == weightsHash && three[1] == graphHash && three[2] == nTensors;
    if (ok)
    {
        _amax.resize(nTensors);
        std::memcpy(_amax.data(), head.data() + header.size() + 1 + sizeof(three), nTensors * sizeof(float));
        const size_t rest = static_cast<size_t>(total) - fixed;
        _file.reset(new unsigned char[rest]);
        ok = std::fread(_file.get(), 1, rest, f) == rest;
        size_t at = 0;
        bool closed = false;
        while (ok && !closed)
        {
            Record r;
            ok = at + sizeof(r) <= rest;
            if (!ok) break;
            std::memcpy(&r, _file.get() + at, sizeof(r));
            at += sizeof(r);
            if (r.op == kClosing)
            {
                closed = true;
                ok = r.algo == _entries.size() && r.bytes == 0 && r.hash == 0 && at == rest;
                break;
            }
            const size_t padded = (static_cast<size_t>(r.bytes) + 7) & ~static_cast<size_t>(7);
            ok = r.bytes <= rest && at + padded <= rest;
            // a blob that does not hash to what was recorded (a flipped bit on disk) must not reach the device as weights
            ok = ok && hash(_file.get() + at, static_cast<size_t>(r.bytes)) == r.hash;
            if (ok) _entries.push_back({r.op, r.algo, at, static_cast<size_t>(r.bytes)});
            at += padded;
        }
        ok = ok && closed;
    }
    std::fclose(f);
    if (!ok)
    {
        _file.reset();
        _entries.clear();
        _amax.clear();
    }
    return ok;
}

const unsigned char *PackFile::blob(uint32_t op, uint32_t algo, size_t bytes)
{
    for (const Entry &e : _entries)
        if (e.op == op)
        {
            if (e.algo != algo || e.bytes != bytes) break;
            ++_served;
            return _file.get() + e.offset;
        }
    _stale = true;
    return nullptr;
}

bool PackFile::create(const std::string &path, const std::string &header, uint64_t weightsHash, uint64_t graphHash, const std::vector<float> &amax)
{
    _path = path;
    _tmp = tempName(path);
    _out = std::fopen(_tmp.c_str(), "wb");
    if (!_out) return false;
    const uint64_t three[3] = {weightsHash, graphHash, amax.size()};
    _failed = std::fwrite(header.data(), 1, header.size(), _out) != header.size() || std::fputc('\n', _out) == EOF ||
              std::fwrite(three, sizeof(uint64_t), 3, _out) != 3 || std::fwrite(amax.data(), sizeof(float), amax.size(), _out) != amax.size();
    return !_failed;
}

void PackFile::add(uint32_t op, uint32_t algo, const void *data, size_t bytes)
{
    if (!_out || _failed) return;
    const Record r = {op, algo, bytes, hash(data, bytes)};
    const unsigned char zeros[8] = {0};
    const size_t pad = ((bytes + 7) & ~static_cast<size_t>(7)) - bytes;
    _failed = std::fwrite(&r, sizeof(r), 1, _out) != 1 || std::fwrite(data, 1, bytes, _out) != bytes || std::fwrite(zeros, 1, pad, _out) != pad;
    ++_written;
}

bool PackFile::commit()
{
    if (!_out) return false;
    const Record r = {kClosing, _written, 0, 0};
    _failed = _failed || std::fwrite(&r, sizeof(r), 1, _out) != 1;
    _failed = std::fclose(_out) != 0 || _failed;
    _out = nullptr;
    if (_failed || std::rename(_tmp.c_str(), _path.c_str()) != 0)
    {
        std::remove(_tmp.c_str());
        return false;
    }
    return true;
}
}
