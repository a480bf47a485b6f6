// File and comparison helpers of the reference's host programs (tests/common/test_common.h: ReadFile :60-110,
// WriteFile :112-150, ResultCmp :211-301), written for this back end's host programs and tests.
#ifndef PTO_HOST_TEST_COMMON_H
#define PTO_HOST_TEST_COMMON_H
#include <cassert>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <iomanip>
#include <iostream> // (the reference's host programs count on this header for their stream output)
#include <string>
#include <vector>

namespace PtoTestCommon {

// Reads at most bufferSize bytes of the file into buffer; fileSize receives the file's size.
inline bool ReadFile(const std::string &path, size_t &fileSize, void *buffer, size_t bufferSize)
{
    FILE *f = std::fopen(path.c_str(), "rb");
    if (f == nullptr) {
        std::fprintf(stderr, "ReadFile: cannot open %s\n", path.c_str());
        return false;
    }
    std::fseek(f, 0, SEEK_END);
    const long size = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (size < 0 || (size_t)size > bufferSize) {
        std::fprintf(stderr, "ReadFile: %s has %ld bytes, the buffer %zu\n", path.c_str(), size, bufferSize);
        std::fclose(f);
        return false;
    }
    const size_t got = std::fread(buffer, 1, (size_t)size, f);
    std::fclose(f);
    fileSize = got;
    return got == (size_t)size;
}

inline bool WriteFile(const std::string &path, const void *buffer, size_t size)
{
    FILE *f = std::fopen(path.c_str(), "wb");
    if (f == nullptr) {
        std::fprintf(stderr, "WriteFile: cannot open %s\n", path.c_str());
        return false;
    }
    const size_t put = std::fwrite(buffer, 1, size, f);
    std::fclose(f);
    return put == size;
}

// An element is wrong when it differs from the expectation by more than eps both absolutely and relatively (or is
// NaN); the comparison passes with at most n * eps wrong elements and at most 1000 results that are zero where the
// expectation is not.
template <typename T>
bool ResultCmp(const std::vector<T> &expect, const T *actual, float eps, size_t count = 0, bool printAll = false)
{
    const size_t n = count ? count : expect.size();
    size_t bad = 0, zeros = 0;
    for (size_t i = 0; i < n; ++i) {
        const float e = (float)expect[i], a = (float)actual[i];
        const float d = std::fabs(e - a), rel = std::fabs(d / e);
        if (std::fabs(a) <= 1e-6f && std::fabs(e) > 1e-6f)
            ++zeros;
        if ((d > eps && rel > eps) || std::isnan(d)) {
            if (bad < 10 || printAll)
                std::fprintf(stderr, "mismatch at %zu: expect %g, got %g\n", i, (double)e, (double)a);
            ++bad;
        }
    }
    return bad <= (size_t)((double)n * eps) && zeros <= 1000;
}
template <typename T>
bool ResultCmp(const std::vector<T> &expect, const std::vector<T> &actual, float eps)
{
    return ResultCmp(expect, actual.data(), eps, expect.size() < actual.size() ? expect.size() : actual.size());
}

} // namespace PtoTestCommon
#endif // PTO_HOST_TEST_COMMON_H
