// Small helpers of the host programs in this directory: whole-file reads and writes, device buffers that free themselves.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <fstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace host_util {

inline void Check(hipError_t e, const char *what)
{
    if (e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// the file's bytes; throws unless it holds exactly `bytes`
inline std::vector<uint8_t> ReadExactly(const std::string &path, size_t bytes)
{
    std::ifstream in(path, std::ios::binary | std::ios::ate);
    if (!in)
        throw std::runtime_error("cannot open " + path);
    const size_t have = (size_t)in.tellg();
    if (have != bytes)
        throw std::runtime_error(path + " holds " + std::to_string(have) + " bytes, expected " + std::to_string(bytes));
    std::vector<uint8_t> data(bytes);
    in.seekg(0);
    in.read(reinterpret_cast<char *>(data.data()), (std::streamsize)bytes);
    if (!in)
        throw std::runtime_error("short read of " + path);
    return data;
}

inline void WriteAll(const std::string &path, const void *data, size_t bytes)
{
    std::ofstream out(path, std::ios::binary | std::ios::trunc);
    out.write(reinterpret_cast<const char *>(data), (std::streamsize)bytes);
    if (!out)
        throw std::runtime_error("cannot write " + path);
}

// device memory for the lifetime of the object, optionally filled from host bytes
class DeviceBuffer {
public:
    explicit DeviceBuffer(size_t bytes) : bytes_(bytes) { Check(hipMalloc(&ptr_, bytes), "hipMalloc"); }
    explicit DeviceBuffer(const std::vector<uint8_t> &host) : DeviceBuffer(host.size())
    {
        Check(hipMemcpy(ptr_, host.data(), host.size(), hipMemcpyHostToDevice), "hipMemcpy to device");
    }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    ~DeviceBuffer() { (void)hipFree(ptr_); }
    template <typename T>
    T *as() const { return static_cast<T *>(ptr_); }
    template <typename T>
    std::vector<T> ToHost() const
    {
        std::vector<T> host(bytes_ / sizeof(T));
        Check(hipMemcpy(host.data(), ptr_, bytes_, hipMemcpyDeviceToHost), "hipMemcpy to host");
        return host;
    }

private:
    void *ptr_ = nullptr;
    size_t bytes_;
};

} // namespace host_util
