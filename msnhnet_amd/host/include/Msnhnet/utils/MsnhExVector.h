// Vector helpers (argsort / maxIndex as in include/Msnhnet/utils/MsnhExVector.h:30-74).
#pragma once
#include <algorithm>
#include <numeric>
#include <vector>

namespace Msnhnet
{
class ExVector
{
public:
    template <typename T> static long long maxIndex(const std::vector<T> &v)
    {
        return std::distance(v.begin(), std::max_element(v.begin(), v.end()));
    }

    template <typename T> static T max(const std::vector<T> &v) { return *std::max_element(v.begin(), v.end()); }

    template <typename T> static bool contains(const std::vector<T> &v, const T &val)
    {
        return std::find(v.begin(), v.end(), val) != v.end();
    }

    // Index permutation that sorts `a`.  Ties keep their original order (the reference's std::sort leaves
    // tie order unspecified).
    template <typename T> static std::vector<int> argsort(const std::vector<T> &a, bool descending = false)
    {
        std::vector<int> idx(a.size());
        std::iota(idx.begin(), idx.end(), 0);
        if (descending)
            std::stable_sort(idx.begin(), idx.end(), [&a](int i, int j) { return a[i] > a[j]; });
        else
            std::stable_sort(idx.begin(), idx.end(), [&a](int i, int j) { return a[i] < a[j]; });
        return idx;
    }
};
}
