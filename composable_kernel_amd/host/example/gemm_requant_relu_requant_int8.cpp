// int8 GEMM with a fused requant-ReLU-requant epilogue, written the way a user of the
// reference writes it (example/14_gemm_xdl_requant_relu_requant): a functor type of the
// user's own, a concrete device operator, MakeArgument / IsSupportedArgument / MakeInvoker /
// Run. The functor below is the user's; ckx::EpilogueOf recognises its shape (two float
// members scaleGemm_, scaleRelu_) and selects the library's fused epilogue.
//
//   usage: example_gemm_requant_relu_requant_int8 [verify init time] [M N K StrideA StrideB StrideC]
//   CKX_EXAMPLE_DUMP=<file> writes the int8 result for an external check.
#include <cstdlib>
#include <iostream>

#include "ckx/device_ops.hpp"
#include "ckx/host_tensor.hpp"

struct RequantReluRequant
{
    RequantReluRequant(float scaleGemm, float scaleRelu) : scaleGemm_(scaleGemm), scaleRelu_(scaleRelu) {}
    float scaleGemm_;
    float scaleRelu_;
};

using PassThrough = ck::tensor_operation::element_wise::PassThrough;
using Row         = ck::tensor_layout::gemm::RowMajor;
using Col         = ck::tensor_layout::gemm::ColumnMajor;

using DeviceGemmInstance = ck::tensor_operation::device::
    DeviceGemmMfma<Row, Col, Row, int8_t, int8_t, int8_t, PassThrough, PassThrough, RequantReluRequant>;

int main(int argc, char* argv[])
{
    bool time_kernel = false;
    int init_method  = 1;
    ck::index_t M = 3840, N = 4096, K = 4096, StrideA = 4096, StrideB = 4096, StrideC = 4096;
    float scale_gemm = 0.03f, scale_relu = 1.0f;
    if(argc == 4 || argc == 10)
    {
        init_method = std::atoi(argv[2]);
        time_kernel = std::atoi(argv[3]);
    }
    if(argc == 10)
    {
        M = std::atoi(argv[4]), N = std::atoi(argv[5]), K = std::atoi(argv[6]);
        StrideA = std::atoi(argv[7]), StrideB = std::atoi(argv[8]), StrideC = std::atoi(argv[9]);
    }
    else if(argc != 1 && argc != 4)
    {
        std::cout << "arg1: verification, arg2: initialization, arg3: time kernel, arg4 to 9: M N K StrideA StrideB StrideC"
                  << std::endl;
        return 1;
    }

    std::vector<int8_t> a((std::size_t)M * StrideA), b((std::size_t)N * StrideB), c((std::size_t)M * StrideC);
    if(init_method)
    {
        ckx::fill_uniform_int8(a, -5, 5, 0xC0FFEE);
        ckx::fill_uniform_int8(b, -5, 5, 0xC0FFEE + 1);
    }
    ckx::DeviceMem a_dev(a.size()), b_dev(b.size()), c_dev(c.size());
    a_dev.ToDevice(a.data());
    b_dev.ToDevice(b.data());

    auto gemm     = DeviceGemmInstance{};
    auto invoker  = gemm.MakeInvoker();
    auto argument = gemm.MakeArgument(static_cast<int8_t*>(a_dev.GetDeviceBuffer()),
                                      static_cast<int8_t*>(b_dev.GetDeviceBuffer()),
                                      static_cast<int8_t*>(c_dev.GetDeviceBuffer()), M, N, K, StrideA, StrideB, StrideC,
                                      PassThrough{}, PassThrough{}, RequantReluRequant{scale_gemm, scale_relu});
    if(!gemm.IsSupportedArgument(argument))
        throw std::runtime_error("wrong! device_gemm with the specified compilation parameters does not support this GEMM problem");

    float ave_time = invoker.Run(argument, ck::StreamConfig{nullptr, time_kernel});
    ckx::hip_check(hipDeviceSynchronize());
    if(time_kernel)
    {
        const double flop = 2.0 * M * N * K, bytes = (double)M * K + (double)K * N + (double)M * N;
        std::cout << "Perf: " << ave_time << " ms, " << flop / 1e9 / ave_time << " TFlops, " << bytes / 1e6 / ave_time
                  << " GB/s, " << gemm.GetTypeString() << std::endl;
    }
    c_dev.FromDevice(c.data());
    if(const char* path = std::getenv("CKX_EXAMPLE_DUMP"))
        ckx::dump_to_file(path, c);
    long sum = 0;
    for(int8_t v : c)
        sum += v;
    std::cout << "sum(C) = " << sum << std::endl;
    return 0;
}
