// Round trip and rejection cases of the pack file (host code only; no device call).  Prints "ok" or the first failed check.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>
#include "Msnhnet/core/MsnhPackFile.h"

using Msnhnet::PackFile;

#define CHECK(c) do { if (!(c)) { std::printf("failed: %s (line %d)\n", #c, __LINE__); return 1; } } while (0)

static std::vector<unsigned char> slurp(const std::string &p)
{
    std::ifstream f(p, std::ios::binary);
    return std::vector<unsigned char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static void spill(const std::string &p, const std::vector<unsigned char> &v, size_t n)
{
    std::ofstream f(p, std::ios::binary | std::ios::trunc);
    f.write(reinterpret_cast<const char *>(v.data()), static_cast<std::streamsize>(n));
}

int main(int argc, char **argv)
{
    if (argc < 2) return 2;
    const std::string path = std::string(argv[1]) + "/w.msnhbin.f16.pack";
    const std::string line = PackFile::headerLine(1, false);
    CHECK(line.rfind("msnhpack 2 layout ", 0) == 0 && line != PackFile::headerLine(1, true) && line != PackFile::headerLine(0, false));

    // the hash sees every byte, the length and the order
    std::vector<unsigned char> data(1000003);
    for (size_t i = 0; i < data.size(); ++i) data[i] = static_cast<unsigned char>(i * 2654435761u >> 13);
    const uint64_t h0 = PackFile::hash(data.data(), data.size());
    CHECK(h0 == PackFile::hash(data.data(), data.size()));
    for (size_t at : {size_t(0), size_t(7), size_t(31), size_t(32), size_t(500000), data.size() - 1})
    {
        data[at] ^= 1;
        CHECK(PackFile::hash(data.data(), data.size()) != h0);
        data[at] ^= 1;
    }
    CHECK(PackFile::hash(data.data(), data.size() - 1) != h0);
    std::swap(data[8], data[16]);
    CHECK(data[8] == data[16] || PackFile::hash(data.data(), data.size()) != h0);
    std::swap(data[8], data[16]);
    const std::vector<unsigned char> zeros(64, 0);
    CHECK(PackFile::hash(zeros.data(), 32) != PackFile::hash(zeros.data(), 64) && PackFile::hash(zeros.data(), 0) != PackFile::hash(zeros.data(), 1));

    const std::vector<float> amax = {0.f, 1.5f, 3e4f, 7.25f};
    {
        PackFile w;
        CHECK(w.create(path, line, 11, 22, amax));
        w.add(3, 2, data.data(), 1001);            // odd size: padded to 8 in the file
        w.add(9, 112, data.data() + 5000, 64);
        CHECK(std::ifstream(path).good() == false); // nothing under the final name before commit
        CHECK(w.commit());
    }
    {
        PackFile r;
        CHECK(r.open(path, line, 11, 22, amax.size()));
        CHECK(r.amax() == amax);
        const unsigned char *a = r.blob(3, 2, 1001), *b = r.blob(9, 112, 64);
        CHECK(a && b && std::memcmp(a, data.data(), 1001) == 0 && std::memcmp(b, data.data() + 5000, 64) == 0 && !r.stale() && r.blobsServed() == 2);
        CHECK(r.blob(3, 4, 1001) == nullptr && r.stale());          // another algorithm
        CHECK(r.blob(9, 112, 72) == nullptr && r.blob(5, 2, 8) == nullptr);
    }
    // what must be refused: other weights, another plan, another tensor count, another library line, a cut file, a missing closing record
    { PackFile r; CHECK(!r.open(path, line, 12, 22, amax.size())); }
    { PackFile r; CHECK(!r.open(path, line, 11, 23, amax.size())); }
    { PackFile r; CHECK(!r.open(path, line, 11, 22, amax.size() + 1)); }
    { PackFile r; CHECK(!r.open(path, PackFile::headerLine(1, true), 11, 22, amax.size())); }
    { PackFile r; CHECK(!r.open(path + ".absent", line, 11, 22, amax.size())); }
    const std::vector<unsigned char> whole = slurp(path);
    for (size_t cut : {whole.size() - 1, whole.size() - 16, whole.size() - 17, whole.size() / 2, line.size() + 5, size_t(3), size_t(0)})
    {
        spill(path, whole, cut);
        PackFile r;
        CHECK(!r.open(path, line, 11, 22, amax.size()));
    }
    {
        std::vector<unsigned char> longer = whole;
        longer.push_back(0);
        spill(path, longer, longer.size());
        PackFile r;
        CHECK(!r.open(path, line, 11, 22, amax.size()));
    }
    // one flipped bit inside a blob: the blob's checksum refuses the whole file
    for (size_t at : {whole.size() - 16 - 24 - 40, whole.size() / 2})
    {
        std::vector<unsigned char> flipped = whole;
        flipped[at] ^= 0x10;
        spill(path, flipped, flipped.size());
        PackFile r;
        CHECK(!r.open(path, line, 11, 22, amax.size()));
    }
    // an abandoned writer leaves neither the file nor its temporary
    std::remove(path.c_str());
    {
        PackFile w;
        CHECK(w.create(path, line, 1, 2, amax));
        w.add(0, 2, data.data(), 100);
    }
    CHECK(!std::ifstream(path).good());
    {
        // (temporaries are named "<path>.tmp.<pid>.<n>": none may be left in the directory)
        const std::string dir = path.substr(0, path.find_last_of('/'));
        const std::string cmd = "ls " + dir + " | grep -c '\\.tmp\\.' > " + dir + "/count.txt";
        (void)std::system(cmd.c_str());
        std::ifstream c(dir + "/count.txt");
        int n = -1;
        c >> n;
        CHECK(n == 0);
    }
    std::printf("ok\n");
    return 0;
}
