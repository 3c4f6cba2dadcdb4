// Host-side harness pieces used by the profiler and the examples: device buffers, seeded
// tensor generators and the check_err comparator. Plays the part of the reference's
// library/include/ck/library/host_tensor/{device_memory.hpp, host_tensor_generator.hpp} and
// library/include/ck/library/utility/check_err.hpp:24-193.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace ckx {

inline void hip_check(hipError_t e, const char* what = "HIP runtime error")
{
    if(e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// library/src/host_tensor/device_memory.cpp:7-28
struct DeviceMem
{
    explicit DeviceMem(std::size_t bytes) : bytes_(bytes) { hip_check(hipMalloc(&p_, bytes ? bytes : 1)); }
    DeviceMem(const DeviceMem&) = delete;
    DeviceMem& operator=(const DeviceMem&) = delete;
    ~DeviceMem() { (void)hipFree(p_); }
    void* GetDeviceBuffer() const { return p_; }
    std::size_t GetBufferSize() const { return bytes_; }
    void ToDevice(const void* src) { hip_check(hipMemcpy(p_, src, bytes_, hipMemcpyHostToDevice)); }
    void FromDevice(void* dst) const { hip_check(hipMemcpy(dst, p_, bytes_, hipMemcpyDeviceToHost)); }
    void SetZero() { hip_check(hipMemset(p_, 0, bytes_)); }
    void* p_ = nullptr;
    std::size_t bytes_;
};

// Counter-based generator: element i depends only on (seed, i); the same mixer as
// composable_kernel_amd/host_tensor.py, so a test can rebuild the profiler's inputs.
inline uint64_t splitmix64(uint64_t seed, uint64_t i)
{
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void fill_uniform_int8(std::vector<int8_t>& v, int lo, int hi, uint64_t seed)
{
    const uint64_t span = (uint64_t)(hi - lo + 1);
    for(std::size_t i = 0; i < v.size(); ++i)
        v[i] = (int8_t)((int64_t)((splitmix64(seed, i) >> 33) % span) + lo);
}

inline void fill_uniform_f16(std::vector<_Float16>& v, float lo, float hi, uint64_t seed)
{
    for(std::size_t i = 0; i < v.size(); ++i)
    {
        const float u = (float)(splitmix64(seed, i) >> 40) * (1.0f / (float)(1 << 24));
        v[i]          = (_Float16)(lo + u * (hi - lo));
    }
}

// bfloat16 bit patterns: widening is a shift, narrowing rounds to nearest even
// (type_convert<bhalf_t, float>, include/ck/utility/data_type.hpp:953-993, finite inputs)
inline float bf16_to_float(unsigned short h)
{
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
inline unsigned short float_to_bf16(float x)
{
    uint32_t u;
    std::memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
inline void fill_uniform_bf16(std::vector<unsigned short>& v, float lo, float hi, uint64_t seed)
{
    for(std::size_t i = 0; i < v.size(); ++i)
    {
        const float u = (float)(splitmix64(seed, i) >> 40) * (1.0f / (float)(1 << 24));
        v[i]          = float_to_bf16(lo + u * (hi - lo));
    }
}
inline std::size_t count_errors(const std::vector<unsigned short>& out, const std::vector<unsigned short>& ref,
                                double rtol, double atol)
{
    std::size_t bad = 0;
    for(std::size_t i = 0; i < ref.size(); ++i)
    {
        const double o = bf16_to_float(out[i]), r = bf16_to_float(ref[i]);
        if(std::fabs(o - r) > atol + rtol * std::fabs(r) || !std::isfinite(o) || !std::isfinite(r))
            ++bad;
    }
    return bad;
}

// |o - r| <= atol + rtol * |r| and finite, as check_err; returns the number of violations
inline std::size_t count_errors(const std::vector<_Float16>& out, const std::vector<_Float16>& ref, double rtol,
                                double atol)
{
    std::size_t bad = 0;
    for(std::size_t i = 0; i < ref.size(); ++i)
    {
        const double o = (double)out[i], r = (double)ref[i];
        if(std::fabs(o - r) > atol + rtol * std::fabs(r) || !std::isfinite(o) || !std::isfinite(r))
            ++bad;
    }
    return bad;
}

inline std::size_t count_errors(const std::vector<int8_t>& out, const std::vector<int8_t>& ref, double, double)
{
    std::size_t bad = 0;
    for(std::size_t i = 0; i < ref.size(); ++i)
        bad += out[i] != ref[i];
    return bad;
}

template <typename T>
void dump_to_file(const char* path, const std::vector<T>& v)
{
    FILE* f = std::fopen(path, "wb");
    if(!f)
        throw std::runtime_error(std::string("cannot write ") + path);
    std::fwrite(v.data(), sizeof(T), v.size(), f);
    std::fclose(f);
}

} // namespace ckx
