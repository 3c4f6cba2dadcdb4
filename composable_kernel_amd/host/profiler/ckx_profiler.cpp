// ckx_profiler: ckProfiler-style driver (profiler/src/profiler.cpp:48-148) for the operators of
// this library. Positional arguments follow the reference's conventions
// (profiler/src/profile_gemm.cpp:27-75, profile_convnd_fwd.cpp:81-115):
//
//   ckx_profiler gemm <dtype 1:fp16 2:bf16 3:int8> <layout 0:mk_kn 1:mk_nk 2:km_kn 3:km_nk> <verify> <init> <log> <time>
//                     M N K StrideA StrideB StrideC [epilogue 0|1|2] [scale_gemm] [scale_relu] [nrepeat]
//   ckx_profiler conv2d_fwd <dtype 1|3> <verify> <init> <log> <time>
//                     N K C Y X Hi Wi Sy Sx Dy Dx LeftPy LeftPx RightPy RightPx [epilogue sg sr] [nrepeat]
//   ckx_profiler convnd_fwd <dtype 1|3> <layout 1> <verify> <init> <log> <nrepeat> <NDim 1|2|3>
//                     N K C <filter> <input> <strides> <dilations> <left pads> <right pads>   (NDim values each)
//   ckx_profiler batched_gemm_gemm <verify> <init> <log> <time> M N K O Batch [nrepeat]
//   ckx_profiler batched_gemm_softmax_gemm <verify> <init> <log> <time> M N K O Batch [scale] [mask 0|1] [nrepeat]
//   ckx_profiler conv_fwd_bias_relu | conv_fwd_bias_relu_add <dtype 1> <verify> <init> <log> <time>
//                     N K C Y X Hi Wi Sy Sx Dy Dx LeftPy LeftPx RightPy RightPx [nrepeat]
//                     (profiler/src/profile_conv_fwd_bias_relu[_add].cpp; fp16, NHWC/KYXC/NHWK)
//   ckx_profiler gemm_splitk <dtype 1|3> <layout 1> <verify> <init> <log> <time> M N K StrideA StrideB StrideC KBatch
//                     [nrepeat]   (profiler/src/profile_gemm_splitk.cpp; PassThrough output)
//   ckx_profiler batched_gemm <dtype 1|3> <layout 1> <verify> <init> <log> <time> M N K StrideA StrideB StrideC
//                     BatchCount [nrepeat]   (profiler/src/profile_batched_gemm.cpp; dense batch strides)
//   ckx_profiler gemm_bias_relu <verify> <init> <log> <time> M N K StrideA StrideB StrideE [nrepeat]
//                     (example/03_gemm_bias_relu: E = AddRelu(half(A*B), bias row), fp16)
//   ckx_profiler gemm_bilinear <dtype 1> <layout 0..3> <verify> <init> <log> <time> M N K StrideA StrideB StrideD StrideE
//                     alpha beta [nrepeat]   (profiler/src/profile_gemm_bilinear.cpp:28-66)
//   ckx_profiler gemm_add_add_fastgelu <dtype 1> <layout 0..3> <verify> <init> <log> <time> M N K StrideA StrideB
//                     StrideD0 StrideD1 StrideE [nrepeat]   (profiler/src/profile_gemm_add_add_fastgelu.cpp:29-62)
//
// Every instance of the family is run (DeviceOperationInstanceFactory), one "Perf:" line each
// and a final "Best Perf:" line, in the reference's format (profile_gemm_impl.hpp:176-177,
// 246-249), extended with the fraction of the MI355X roofline that binds the problem.
// verify = 1 checks that all instances agree with the first supported one (bit-exact for
// int8, rtol = atol = 1e-2 for fp16); comparison against the CPU reference is the job of the
// test-suite, which regenerates these inputs from the same seeds. If the environment variable
// CKX_PROFILER_DUMP names a file, the best instance's output tensor is written there.
#include <cstdlib>
#include <cstring>
#include <iomanip>
#include <iostream>

#include "ckx/device_ops.hpp"
#include "ckx/host_tensor.hpp"

using namespace ck;
using namespace ck::tensor_operation;
using Row  = tensor_layout::gemm::RowMajor;
using Col  = tensor_layout::gemm::ColumnMajor;
using Pass = element_wise::PassThrough;

namespace {

constexpr double kPeakF16 = 2516.6, kPeakI8 = 5033.2, kPeakHbmGBs = 8000.0;

struct Best
{
    float ms = 0, tflops = 0, gbs = 0;
    std::string name;
    int id = -1;
};

void report(const char* tag, float ms, double flop, double bytes, const std::string& name, bool i8)
{
    const double tflops = flop / 1e9 / ms, gbs = bytes / 1e6 / ms;
    const double fm = tflops / (i8 ? kPeakI8 : kPeakF16), fh = gbs / kPeakHbmGBs;
    std::cout << tag << std::setw(10) << ms << " ms, " << tflops << " TFlops, " << gbs << " GB/s, " << name << "  ["
              << std::fixed << std::setprecision(1) << (fm >= fh ? fm : fh) * 100 << "% of "
              << (fm >= fh ? "MFMA" : "HBM") << " roofline]" << std::defaultfloat << std::setprecision(6)
              << std::endl;
}

template <typename T>
void fill(std::vector<T>& v, int init, uint64_t seed, bool conv)
{
    if constexpr(std::is_same_v<T, int8_t>)
    {
        if(init == 0)
            return;
        ckx::fill_uniform_int8(v, -5, 5, seed);
    }
    else if constexpr(std::is_same_v<T, bhalf_t>)
    {
        if(init == 0)
            return;
        if(init == 1)
        {
            std::vector<int8_t> t(v.size());
            ckx::fill_uniform_int8(t, -5, 5, seed);
            for(std::size_t i = 0; i < v.size(); ++i)
                v[i] = ckx::float_to_bf16((float)t[i]);
        }
        else
            ckx::fill_uniform_bf16(v, -1.f, 1.f, seed);
    }
    else
    {
        if(init == 0)
            return;
        if(init == 1)
        { // integer values, as the reference's init_method 1
            std::vector<int8_t> t(v.size());
            ckx::fill_uniform_int8(t, -5, 5, seed);
            for(std::size_t i = 0; i < v.size(); ++i)
                v[i] = (T)(float)t[i];
        }
        else
            ckx::fill_uniform_f16(v, conv ? -1.f : -1.f, 1.f, seed);
    }
}

template <typename T, typename Op, typename MakeArg>
int run_family(std::vector<std::unique_ptr<Op>>& ops, MakeArg make_arg, ckx::DeviceMem& out_dev, std::size_t out_elems,
               double flop, double bytes, bool verify, bool time_kernel, int nrepeat)
{
    constexpr bool i8 = std::is_same_v<T, int8_t>;
    std::cout << "found " << ops.size() << " instances" << std::endl;
    Best best;
    std::vector<T> ref, out(out_elems);
    bool pass = true;
    for(std::size_t i = 0; i < ops.size(); ++i)
    {
        auto arg = make_arg(*ops[i]);
        auto inv = ops[i]->MakeInvokerPointer();
        const std::string name = ops[i]->GetTypeString();
        if(!ops[i]->IsSupportedArgument(arg.get()))
        {
            std::cout << name << " does not support this problem" << std::endl;
            continue;
        }
        out_dev.SetZero();
        StreamConfig sc{nullptr, time_kernel, nrepeat, nrepeat >= 100 ? nrepeat / 4 : 1};
        const float ms = inv->Run(arg.get(), sc);
        ckx::hip_check(hipDeviceSynchronize());
        if(time_kernel)
        {
            report("Perf: ", ms, flop, bytes, name, i8);
            if(best.id < 0 || ms < best.ms)
                best = Best{ms, (float)(flop / 1e9 / ms), (float)(bytes / 1e6 / ms), name, (int)i};
        }
        else if(best.id < 0)
            best.id = (int)i, best.name = name;
        if(verify)
        {
            out_dev.FromDevice(out.data());
            if(ref.empty())
                ref = out;
            else
            {
                const std::size_t bad = ckx::count_errors(out, ref, 1e-2, 1e-2);
                if(bad)
                {
                    std::cout << "Error: " << name << " disagrees with the first instance on " << bad << " elements"
                              << std::endl;
                    pass = false;
                }
            }
        }
    }
    if(best.id < 0)
    {
        std::cout << "no instance supports this problem" << std::endl;
        return 1;
    }
    if(time_kernel)
        report("Best Perf: ", best.ms, flop, bytes, best.name, i8);
    if(const char* path = std::getenv("CKX_PROFILER_DUMP"))
    {
        auto arg = make_arg(*ops[best.id]);
        out_dev.SetZero();
        ops[best.id]->MakeInvokerPointer()->Run(arg.get(), StreamConfig{});
        ckx::hip_check(hipDeviceSynchronize());
        out_dev.FromDevice(out.data());
        ckx::dump_to_file(path, out);
    }
    return pass ? 0 : 1;
}

// layout codes of the reference's profiler (profiler/src/profile_gemm.cpp:13-19)
enum GemmMatrixLayout
{
    MK_KN_MN = 0,
    MK_NK_MN = 1,
    KM_KN_MN = 2,
    KM_NK_MN = 3
};

template <typename T, typename COp, typename AL, typename BL>
int profile_gemm_l(bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sc, COp cop,
                   int nrepeat)
{
    using DeviceOp = device::DeviceGemm<AL, BL, Row, T, T, T, Pass, Pass, COp>;
    auto ops       = device::instance::DeviceOperationInstanceFactory<DeviceOp>::GetInstances();
    constexpr bool a_row = std::is_same_v<AL, Row>, b_row = std::is_same_v<BL, Row>;
    sa = sa < 0 ? (a_row ? K : M) : sa, sb = sb < 0 ? (b_row ? N : K) : sb, sc = sc < 0 ? N : sc;
    std::vector<T> a((std::size_t)(a_row ? M : K) * sa), b((std::size_t)(b_row ? K : N) * sb);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    ckx::DeviceMem da(a.size() * sizeof(T)), db(b.size() * sizeof(T)), dc((std::size_t)M * sc * sizeof(T));
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    std::cout << "a_m_k: dim 2, lengths {" << M << ", " << K << "}, strides {" << (a_row ? sa : 1) << ", "
              << (a_row ? 1 : sa) << "}\n"
              << "b_k_n: dim 2, lengths {" << K << ", " << N << "}, strides {" << (b_row ? sb : 1) << ", "
              << (b_row ? 1 : sb) << "}\n"
              << "c_m_n: dim 2, lengths {" << M << ", " << N << "}, strides {" << sc << ", 1}" << std::endl;
    const double flop = 2.0 * M * N * K, bytes = sizeof(T) * ((double)M * K + (double)K * N + (double)M * N);
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), dc.GetDeviceBuffer(), M, N, K,
                                          sa, sb, sc, Pass{}, Pass{}, cop);
        },
        dc, (std::size_t)M * sc, flop, bytes, verify, time_kernel, nrepeat);
}

template <typename T, typename COp>
int profile_gemm_t(int layout, bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sc,
                   COp cop, int nrepeat)
{
    switch(layout)
    {
    case MK_KN_MN: return profile_gemm_l<T, COp, Row, Row>(verify, init, time_kernel, M, N, K, sa, sb, sc, cop, nrepeat);
    case MK_NK_MN: return profile_gemm_l<T, COp, Row, Col>(verify, init, time_kernel, M, N, K, sa, sb, sc, cop, nrepeat);
    case KM_KN_MN: return profile_gemm_l<T, COp, Col, Row>(verify, init, time_kernel, M, N, K, sa, sb, sc, cop, nrepeat);
    case KM_NK_MN: return profile_gemm_l<T, COp, Col, Col>(verify, init, time_kernel, M, N, K, sa, sb, sc, cop, nrepeat);
    }
    std::cout << "this data_type & layout is not implemented" << std::endl;
    return 1;
}

int profile_gemm(int argc, char* argv[])
{
    if(argc < 14)
    {
        std::printf("arg1: tensor operation (gemm)\narg2: data type (1: fp16; 2: bf16; 3: int8)\n"
                    "arg3: matrix layout (0: A[m, k] * B[k, n] = C[m, n];\n"
                    "                     1: A[m, k] * B[n, k] = C[m, n];\n"
                    "                     2: A[k, m] * B[k, n] = C[m, n];\n"
                    "                     3: A[k, m] * B[n, k] = C[m, n])\n"
                    "arg4: verification (0: no; 1: yes)\n"
                    "arg5: initialization (0: no init; 1: integer value; 2: decimal value)\n"
                    "arg6: print tensor value (0: no; 1: yes)\narg7: time kernel (0=no, 1=yes)\n"
                    "arg8 to 13: M, N, K, StrideA, StrideB, StrideC (negative: packed)\n"
                    "arg14-16 (int8): epilogue (0 PassThrough, 1 RequantReluRequant, 2 rounded), scale_gemm, scale_relu\n"
                    "last: nrepeat\n");
        return 1;
    }
    const int dtype = std::atoi(argv[2]), layout = std::atoi(argv[3]);
    const bool verify = std::atoi(argv[4]), time_kernel = std::atoi(argv[7]);
    const int init = std::atoi(argv[5]);
    const int M = std::atoi(argv[8]), N = std::atoi(argv[9]), K = std::atoi(argv[10]);
    int sa = std::atoi(argv[11]), sb = std::atoi(argv[12]), sc = std::atoi(argv[13]);
    if(dtype == 1)
        return profile_gemm_t<half_t>(layout, verify, init, time_kernel, M, N, K, sa, sb, sc, Pass{},
                                      argc > 14 ? std::atoi(argv[14]) : 10);
    if(dtype == 2)
        return profile_gemm_t<bhalf_t>(layout, verify, init, time_kernel, M, N, K, sa, sb, sc, Pass{},
                                       argc > 14 ? std::atoi(argv[14]) : 10);
    if(dtype == 3)
    {
        const int epi  = argc > 14 ? std::atoi(argv[14]) : 0;
        const float sg = argc > 15 ? (float)std::atof(argv[15]) : 0.03f;
        const float sr = argc > 16 ? (float)std::atof(argv[16]) : 1.0f;
        const int nrep = argc > 17 ? std::atoi(argv[17]) : 10;
        if(epi == 0)
            return profile_gemm_t<int8_t>(layout, verify, init, time_kernel, M, N, K, sa, sb, sc, Pass{}, nrep);
        if(epi == 1)
            return profile_gemm_t<int8_t>(layout, verify, init, time_kernel, M, N, K, sa, sb, sc,
                                          element_wise::RequantReluRequant{sg, sr}, nrep);
        return profile_gemm_t<int8_t>(layout, verify, init, time_kernel, M, N, K, sa, sb, sc,
                                      element_wise::RequantRoundReluRequantRound{sg, sr}, nrep);
    }
    std::cout << "this data_type & layout is not implemented" << std::endl;
    return 1;
}

template <typename T, typename OutOp>
int profile_conv_t(bool verify, int init, bool time_kernel, const int* p, OutOp oop, int nrepeat)
{
    const int N = p[0], K = p[1], C = p[2], Y = p[3], X = p[4], Hi = p[5], Wi = p[6], Sy = p[7], Sx = p[8],
              Dy = p[9], Dx = p[10], LPy = p[11], LPx = p[12], RPy = p[13], RPx = p[14];
    // conv_util.cpp:103-114
    const int Ho = (Hi + LPy + RPy - ((Y - 1) * Dy + 1)) / Sy + 1, Wo = (Wi + LPx + RPx - ((X - 1) * Dx + 1)) / Sx + 1;
    auto ops     = device::instance::GetConv2dFwdInstances<T, Pass, Pass, OutOp>();
    using Op     = device::DeviceConvFwd<Pass, Pass, OutOp>;
    std::vector<T> in((std::size_t)N * Hi * Wi * C), wei((std::size_t)K * Y * X * C);
    fill(in, init, 0xC0FFEE + 2, true);
    fill(wei, init, 0xC0FFEE + 3, true);
    const std::size_t out_elems = (std::size_t)N * Ho * Wo * K;
    ckx::DeviceMem di(in.size() * sizeof(T)), dw(wei.size() * sizeof(T)), dout(out_elems * sizeof(T));
    di.ToDevice(in.data());
    dw.ToDevice(wei.data());
    std::cout << "input: N " << N << " Hi " << Hi << " Wi " << Wi << " C " << C << "; weight: K " << K << " Y " << Y
              << " X " << X << "; output: Ho " << Ho << " Wo " << Wo << std::endl;
    // conv_util.cpp:22-39 (flops) and conv_util.hpp:108-136 (bytes: whole input counted)
    const double flop  = 2.0 * N * K * Ho * Wo * C * Y * X;
    const double bytes = sizeof(T) * ((double)in.size() + (double)wei.size() + (double)out_elems);
    return run_family<T>(
        ops,
        [&](Op& op) {
            return op.MakeArgumentPointer(di.GetDeviceBuffer(), dw.GetDeviceBuffer(), dout.GetDeviceBuffer(), N, K, C,
                                          {Hi, Wi}, {Y, X}, {Ho, Wo}, {Sy, Sx}, {Dy, Dx}, {LPy, LPx}, {RPy, RPx},
                                          Pass{}, Pass{}, oop);
        },
        dout, out_elems, flop, bytes, verify, time_kernel, nrepeat);
}

int profile_conv(int argc, char* argv[])
{
    if(argc < 22)
    {
        std::printf("arg1: tensor operation (conv2d_fwd)\narg2: data type (1: fp16; 3: int8)\n"
                    "arg3: verification\narg4: initialization\narg5: print tensor value\narg6: time kernel\n"
                    "arg7 to 21: N, K, C, Y, X, Hi, Wi, Sy, Sx, Dy, Dx, LeftPy, LeftPx, RightPy, RightPx\n"
                    "arg22-24 (int8): epilogue, scale_gemm, scale_relu; last: nrepeat\n");
        return 1;
    }
    const int dtype = std::atoi(argv[2]);
    const bool verify = std::atoi(argv[3]), time_kernel = std::atoi(argv[6]);
    const int init = std::atoi(argv[4]);
    int p[15];
    for(int i = 0; i < 15; ++i)
        p[i] = std::atoi(argv[7 + i]);
    if(dtype == 1)
        return profile_conv_t<half_t>(verify, init, time_kernel, p, Pass{}, argc > 22 ? std::atoi(argv[22]) : 10);
    if(dtype == 3)
    {
        const int epi  = argc > 22 ? std::atoi(argv[22]) : 0;
        const float sg = argc > 23 ? (float)std::atof(argv[23]) : 0.03f;
        const float sr = argc > 24 ? (float)std::atof(argv[24]) : 1.0f;
        const int nrep = argc > 25 ? std::atoi(argv[25]) : 10;
        if(epi == 0)
            return profile_conv_t<int8_t>(verify, init, time_kernel, p, Pass{}, nrep);
        if(epi == 1)
            return profile_conv_t<int8_t>(verify, init, time_kernel, p, element_wise::RequantReluRequant{sg, sr}, nrep);
        return profile_conv_t<int8_t>(verify, init, time_kernel, p, element_wise::RequantRoundReluRequantRound{sg, sr},
                                      nrep);
    }
    std::cout << "this data_type is not implemented" << std::endl;
    return 1;
}

// conv forward with NDim spatial dimensions, channels-last tensors
// (profiler/src/profile_convnd_fwd.cpp:81-115: N, K, C, then filter / input / strides / dilations / left pads /
// right pads, NDim values each)
template <int NDim, typename T, typename OutOp>
int profile_convnd_t(bool verify, int init, bool time_kernel, const int* p, OutOp oop, int nrepeat)
{
    const int N = p[0], K = p[1], C = p[2];
    std::vector<index_t> filt(p + 3, p + 3 + NDim), in_len(p + 3 + NDim, p + 3 + 2 * NDim),
        st(p + 3 + 2 * NDim, p + 3 + 3 * NDim), dl(p + 3 + 3 * NDim, p + 3 + 4 * NDim),
        lp(p + 3 + 4 * NDim, p + 3 + 5 * NDim), rp(p + 3 + 5 * NDim, p + 3 + 6 * NDim), out_len(NDim);
    std::size_t in_px = N, out_px = N, taps = 1;
    for(int i = 0; i < NDim; ++i)
    {
        // conv_util.cpp:103-114
        out_len[i] = (in_len[i] + lp[i] + rp[i] - ((filt[i] - 1) * dl[i] + 1)) / st[i] + 1;
        in_px *= in_len[i], out_px *= out_len[i] > 0 ? out_len[i] : 0, taps *= filt[i];
    }
    auto ops = device::instance::GetConvNdFwdInstances<NDim, T, Pass, Pass, OutOp>();
    using Op = device::DeviceConvFwd<Pass, Pass, OutOp>;
    std::vector<T> in(in_px * C), wei((std::size_t)K * taps * C);
    fill(in, init, 0xC0FFEE + 2, true);
    fill(wei, init, 0xC0FFEE + 3, true);
    const std::size_t out_elems = out_px * K;
    ckx::DeviceMem di(in.size() * sizeof(T)), dw(wei.size() * sizeof(T)), dout(out_elems * sizeof(T));
    di.ToDevice(in.data());
    dw.ToDevice(wei.data());
    std::cout << NDim << " spatial dimensions; N " << N << " K " << K << " C " << C << "; output pixels per image "
              << out_px / (N ? N : 1) << std::endl;
    const double flop  = 2.0 * (double)out_px * K * C * (double)taps; // conv_util.cpp:22-39
    const double bytes = sizeof(T) * ((double)in.size() + (double)wei.size() + (double)out_elems);
    return run_family<T>(
        ops,
        [&](Op& op) {
            return op.MakeArgumentPointer(di.GetDeviceBuffer(), dw.GetDeviceBuffer(), dout.GetDeviceBuffer(), N, K, C,
                                          in_len, filt, out_len, st, dl, lp, rp, Pass{}, Pass{}, oop);
        },
        dout, out_elems, flop, bytes, verify, time_kernel, nrepeat);
}

template <int NDim>
int profile_convnd_dim(int dtype, bool verify, int init, bool time_kernel, const int* p, int nrepeat)
{
    if(dtype == 1)
        return profile_convnd_t<NDim, half_t>(verify, init, time_kernel, p, Pass{}, nrepeat);
    if(dtype == 3)
        return profile_convnd_t<NDim, int8_t>(verify, init, time_kernel, p, Pass{}, nrepeat);
    std::cout << "this data_type is not implemented" << std::endl;
    return 1;
}

int profile_convnd(int argc, char* argv[])
{
    const int ndim = argc > 8 ? std::atoi(argv[8]) : 0;
    if(ndim < 1 || ndim > 3 || argc != 9 + 3 + 6 * ndim)
    {
        std::printf("arg1: tensor operation (convnd_fwd)\narg2: data type (1: fp16; 3: int8)\n"
                    "arg3: data layout (1: channels last)\narg4: verification\narg5: initialization\n"
                    "arg6: print tensor value\narg7: run kernel # of times\narg8: N spatial dimensions (1, 2, 3)\n"
                    "then N, K, C, <filter>, <input>, <strides>, <dilations>, <left pads>, <right pads>\n");
        return 1;
    }
    if(std::atoi(argv[3]) != 1)
    {
        std::cout << "this data layout is not implemented" << std::endl;
        return 1;
    }
    const int dtype = std::atoi(argv[2]), init = std::atoi(argv[5]), nrep = std::atoi(argv[7]);
    const bool verify = std::atoi(argv[4]);
    int p[3 + 18];
    for(int i = 0; i < 3 + 6 * ndim; ++i)
        p[i] = std::atoi(argv[9 + i]);
    const bool time_kernel = nrep > 0;
    if(ndim == 1)
        return profile_convnd_dim<1>(dtype, verify, init, time_kernel, p, nrep > 0 ? nrep : 1);
    if(ndim == 2)
        return profile_convnd_dim<2>(dtype, verify, init, time_kernel, p, nrep > 0 ? nrep : 1);
    return profile_convnd_dim<3>(dtype, verify, init, time_kernel, p, nrep > 0 ? nrep : 1);
}

template <typename T>
int profile_gemm_splitk_t(bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sc,
                          int kbatch, int nrepeat)
{
    using DeviceOp = device::DeviceGemmSplitK<Row, Col, Row, T, T, T, Pass, Pass, Pass>;
    std::vector<std::unique_ptr<DeviceOp>> ops;
    for(int i = 0, n = ckx_num_instances(CKX_OP_GEMM_SPLITK); i < n; ++i)
        ops.push_back(std::make_unique<device::DeviceGemmSplitKMfma<Row, Col, Row, T, T, T, Pass, Pass, Pass>>(i));
    std::vector<T> a((std::size_t)M * sa), b((std::size_t)N * sb);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    ckx::DeviceMem da(a.size() * sizeof(T)), db(b.size() * sizeof(T)), dc((std::size_t)M * sc * sizeof(T));
    const int op_code = std::is_same_v<T, int8_t> ? CKX_OP_GEMM_I8 : CKX_OP_GEMM_F16;
    ckx::DeviceMem ws((std::size_t)ckx_gemm_splitk_workspace_bytes(op_code, M, N, K, kbatch) + 16);
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    const double flop = 2.0 * M * N * K, bytes = sizeof(T) * ((double)M * K + (double)K * N + (double)M * N);
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            auto arg = op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), dc.GetDeviceBuffer(), M, N,
                                              K, sa, sb, sc, Pass{}, Pass{}, Pass{}, kbatch);
            op.SetWorkSpacePointer(arg.get(), ws.GetDeviceBuffer());
            return arg;
        },
        dc, (std::size_t)M * sc, flop, bytes, verify, time_kernel, nrepeat);
}

int profile_gemm_splitk(int argc, char* argv[])
{
    if(argc < 15)
    {
        std::printf("arg1: tensor operation (gemm_splitk)\narg2: data type (1: fp16; 3: int8)\n"
                    "arg3: matrix layout (1: A[m, k] * B[n, k] = C[m, n])\narg4: verification\n"
                    "arg5: initialization\narg6: print tensor value\narg7: time kernel\n"
                    "arg8 to 13: M, N, K, StrideA, StrideB, StrideC\narg14: split k into multiple batch\n");
        return 1;
    }
    const int dtype = std::atoi(argv[2]), layout = std::atoi(argv[3]);
    const bool verify = std::atoi(argv[4]), time_kernel = std::atoi(argv[7]);
    const int init = std::atoi(argv[5]);
    const int M = std::atoi(argv[8]), N = std::atoi(argv[9]), K = std::atoi(argv[10]);
    int sa = std::atoi(argv[11]), sb = std::atoi(argv[12]), sc = std::atoi(argv[13]);
    sa = sa < 0 ? K : sa, sb = sb < 0 ? K : sb, sc = sc < 0 ? N : sc;
    const int kbatch = std::atoi(argv[14]), nrep = argc > 15 ? std::atoi(argv[15]) : 10;
    if(layout != 1 || (dtype != 1 && dtype != 3))
    {
        std::cout << "this data_type & layout is not implemented" << std::endl;
        return 1;
    }
    return dtype == 1 ? profile_gemm_splitk_t<half_t>(verify, init, time_kernel, M, N, K, sa, sb, sc, kbatch, nrep)
                      : profile_gemm_splitk_t<int8_t>(verify, init, time_kernel, M, N, K, sa, sb, sc, kbatch, nrep);
}

template <typename T>
int profile_batched_gemm_t(bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sc,
                           int batch, int nrepeat)
{
    using DeviceOp = device::DeviceBatchedGemm<Row, Col, Row, T, T, T, Pass, Pass, Pass>;
    std::vector<std::unique_ptr<DeviceOp>> ops;
    for(int i = 0, n = ckx_num_instances(CKX_OP_GEMM_SPLITK); i < n; ++i) // the tile instances
        ops.push_back(std::make_unique<device::DeviceBatchedGemmMfma<Row, Col, Row, T, T, T, Pass, Pass, Pass>>(i));
    const std::size_t bsa = (std::size_t)M * sa, bsb = (std::size_t)N * sb, bsc = (std::size_t)M * sc;
    std::vector<T> a(bsa * batch), b(bsb * batch);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    ckx::DeviceMem da(a.size() * sizeof(T)), db(b.size() * sizeof(T)), dc(bsc * batch * sizeof(T));
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    const double flop  = 2.0 * M * N * K * batch;
    const double bytes = sizeof(T) * ((double)M * K + (double)K * N + (double)M * N) * batch;
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), dc.GetDeviceBuffer(), M, N, K,
                                          sa, sb, sc, (index_t)bsa, (index_t)bsb, (index_t)bsc, batch, Pass{}, Pass{},
                                          Pass{});
        },
        dc, bsc * batch, flop, bytes, verify, time_kernel, nrepeat);
}

int profile_batched_gemm(int argc, char* argv[])
{
    if(argc < 15)
    {
        std::printf("arg1: tensor operation (batched_gemm)\narg2: data type (1: fp16; 3: int8)\n"
                    "arg3: matrix layout (1: A[g, m, k] * B[g, n, k] = C[g, m, n])\narg4: verification\n"
                    "arg5: initialization\narg6: print tensor value\narg7: time kernel\n"
                    "arg8 to 14: M, N, K, StrideA, StrideB, StrideC, BatchCount\n");
        return 1;
    }
    const int dtype = std::atoi(argv[2]), layout = std::atoi(argv[3]);
    const bool verify = std::atoi(argv[4]), time_kernel = std::atoi(argv[7]);
    const int init = std::atoi(argv[5]);
    const int M = std::atoi(argv[8]), N = std::atoi(argv[9]), K = std::atoi(argv[10]);
    int sa = std::atoi(argv[11]), sb = std::atoi(argv[12]), sc = std::atoi(argv[13]);
    sa = sa < 0 ? K : sa, sb = sb < 0 ? K : sb, sc = sc < 0 ? N : sc;
    const int batch = std::atoi(argv[14]), nrep = argc > 15 ? std::atoi(argv[15]) : 10;
    if(layout != 1 || (dtype != 1 && dtype != 3))
    {
        std::cout << "this data_type & layout is not implemented" << std::endl;
        return 1;
    }
    return dtype == 1 ? profile_batched_gemm_t<half_t>(verify, init, time_kernel, M, N, K, sa, sb, sc, batch, nrep)
                      : profile_batched_gemm_t<int8_t>(verify, init, time_kernel, M, N, K, sa, sb, sc, batch, nrep);
}

// conv + bias + ReLU (with_resi: + residual add), fp16
int profile_conv_bias_relu(int argc, char* argv[], bool with_resi)
{
    if(argc < 22 || std::atoi(argv[2]) != 1)
    {
        std::printf("arg1: tensor operation (conv_fwd_bias_relu[_add])\narg2: data type (1: fp16)\n"
                    "arg3: verification\narg4: initialization\narg5: print tensor value\narg6: time kernel\n"
                    "arg7 to 21: N, K, C, Y, X, Hi, Wi, Sy, Sx, Dy, Dx, LeftPy, LeftPx, RightPy, RightPx\n"
                    "arg22: nrepeat\n");
        return 1;
    }
    using T = half_t;
    const bool verify = std::atoi(argv[3]), time_kernel = std::atoi(argv[6]);
    const int init = std::atoi(argv[4]), nrepeat = argc > 22 ? std::atoi(argv[22]) : 10;
    int p[15];
    for(int i = 0; i < 15; ++i)
        p[i] = std::atoi(argv[7 + i]);
    const int N = p[0], K = p[1], C = p[2], Y = p[3], X = p[4], Hi = p[5], Wi = p[6], Sy = p[7], Sx = p[8],
              Dy = p[9], Dx = p[10], LPy = p[11], LPx = p[12], RPy = p[13], RPx = p[14];
    const int Ho = (Hi + LPy + RPy - ((Y - 1) * Dy + 1)) / Sy + 1, Wo = (Wi + LPx + RPx - ((X - 1) * Dx + 1)) / Sx + 1;
    const std::size_t out_elems = (std::size_t)N * Ho * Wo * K;
    std::vector<T> in((std::size_t)N * Hi * Wi * C), wei((std::size_t)K * Y * X * C), bias((std::size_t)K),
        resi(out_elems);
    fill(in, init, 0xC0FFEE + 2, true);
    fill(wei, init, 0xC0FFEE + 3, true);
    fill(bias, init, 0xC0FFEE + 7, true);
    fill(resi, init, 0xC0FFEE + 8, true);
    ckx::DeviceMem di(in.size() * sizeof(T)), dw(wei.size() * sizeof(T)), db(bias.size() * sizeof(T)),
        dr(resi.size() * sizeof(T)), dout(out_elems * sizeof(T));
    di.ToDevice(in.data());
    dw.ToDevice(wei.data());
    db.ToDevice(bias.data());
    dr.ToDevice(resi.data());
    std::cout << "input: N " << N << " Hi " << Hi << " Wi " << Wi << " C " << C << "; weight: K " << K << " Y " << Y
              << " X " << X << "; output: Ho " << Ho << " Wo " << Wo << std::endl;
    const double flop  = 2.0 * N * K * Ho * Wo * C * Y * X;
    const double bytes = sizeof(T) * ((double)in.size() + (double)wei.size() + (double)K +
                                      (double)out_elems * (with_resi ? 2 : 1));
    if(with_resi)
    {
        using Op = device::DeviceConvFwdBiasActivationAdd<Pass, Pass, element_wise::AddReluAdd>;
        auto ops = device::instance::DeviceOperationInstanceFactory<Op>::GetInstances();
        return run_family<T>(
            ops,
            [&](Op& op) {
                return op.MakeArgumentPointer(di.GetDeviceBuffer(), dw.GetDeviceBuffer(), dout.GetDeviceBuffer(),
                                              db.GetDeviceBuffer(), dr.GetDeviceBuffer(), N, K, C, {Hi, Wi}, {Y, X},
                                              {Ho, Wo}, {Sy, Sx}, {Dy, Dx}, {LPy, LPx}, {RPy, RPx}, Pass{}, Pass{},
                                              element_wise::AddReluAdd{});
            },
            dout, out_elems, flop, bytes, verify, time_kernel, nrepeat);
    }
    using Op = device::DeviceConvFwdBiasActivation<Pass, Pass, element_wise::AddRelu>;
    auto ops = device::instance::DeviceOperationInstanceFactory<Op>::GetInstances();
    return run_family<T>(
        ops,
        [&](Op& op) {
            return op.MakeArgumentPointer(di.GetDeviceBuffer(), dw.GetDeviceBuffer(), dout.GetDeviceBuffer(),
                                          db.GetDeviceBuffer(), N, K, C, {Hi, Wi}, {Y, X}, {Ho, Wo}, {Sy, Sx}, {Dy, Dx},
                                          {LPy, LPx}, {RPy, RPx}, Pass{}, Pass{}, element_wise::AddRelu{});
        },
        dout, out_elems, flop, bytes, verify, time_kernel, nrepeat);
}

// E = AddRelu(half(A * B), D) with D a bias row (stride 0), as example 03 sets it up
int profile_gemm_bias_relu(int argc, char* argv[])
{
    if(argc < 9)
    {
        std::printf("arg1: tensor operation (gemm_bias_relu)\narg2: verification\narg3: initialization\n"
                    "arg4: print tensor value\narg5: time kernel\narg6 to 11: M, N, K, StrideA, StrideB, StrideE\n"
                    "arg12: nrepeat\n");
        return 1;
    }
    using T = half_t;
    const bool verify = std::atoi(argv[2]), time_kernel = std::atoi(argv[5]);
    const int init = std::atoi(argv[3]);
    const int M = std::atoi(argv[6]), N = std::atoi(argv[7]), K = std::atoi(argv[8]);
    int sa = argc > 9 ? std::atoi(argv[9]) : -1, sb = argc > 10 ? std::atoi(argv[10]) : -1,
        se = argc > 11 ? std::atoi(argv[11]) : -1;
    sa = sa < 0 ? K : sa, sb = sb < 0 ? K : sb, se = se < 0 ? N : se;
    const int nrepeat = argc > 12 ? std::atoi(argv[12]) : 10;
    using Ds       = ck::Tuple<T>;
    using DeviceOp = device::DeviceGemmMultipleD<Row, Col, Row, T, T, Ds, T, Pass, Pass, element_wise::AddRelu>;
    auto ops       = device::instance::DeviceOperationInstanceFactory<DeviceOp>::GetInstances();
    std::vector<T> a((std::size_t)M * sa), b((std::size_t)N * sb), d((std::size_t)N);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    fill(d, init, 0xC0FFEE + 9, false);
    ckx::DeviceMem da(a.size() * sizeof(T)), db(b.size() * sizeof(T)), dd(d.size() * sizeof(T)),
        de((std::size_t)M * se * sizeof(T));
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    dd.ToDevice(d.data());
    const double flop = 2.0 * M * N * K, bytes = sizeof(T) * ((double)M * K + (double)K * N + (double)M * N + N);
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), {dd.GetDeviceBuffer()},
                                          de.GetDeviceBuffer(), M, N, K, sa, sb, {0}, se, Pass{}, Pass{},
                                          element_wise::AddRelu{});
        },
        de, (std::size_t)M * se, flop, bytes, verify, time_kernel, nrepeat);
}

// gemm_perchannel_quant <verify> <init> <log> <time> M N K StrideA StrideB StrideE [activation: 0 PassThrough, 1 Relu] [nrepeat]
// int8 A[m,k] * B[n,k] with one fp32 requant scale per output column (the D operand) and Activation_Mul2_Clamp
template <typename Act>
int profile_gemm_perchannel_quant_t(bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int se,
                                    int nrepeat)
{
    using T        = int8_t;
    using CDE      = element_wise::Activation_Mul2_Clamp<Act>;
    using DeviceOp = device::DeviceGemmMultipleD<Row, Col, Row, T, T, ck::Tuple<float>, T, Pass, Pass, CDE>;
    std::vector<std::unique_ptr<DeviceOp>> ops;
    for(int i = 0; i < ckx_num_instances(CKX_OP_GEMM_I8); ++i)
        ops.push_back(std::make_unique<device::DeviceGemmMultipleDInt8Mfma<Row, Col, Row, Act>>(i));
    std::vector<T> a((std::size_t)M * sa), b((std::size_t)N * sb);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    std::vector<float> scale((std::size_t)N);
    for(int n = 0; n < N; ++n) // a different, exactly representable scale per column, both signs
        scale[n] = (float)((n * 37) % 61 - 20) / 256.0f;
    ckx::DeviceMem da(a.size()), db(b.size()), dd(scale.size() * sizeof(float)), de((std::size_t)M * se);
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    dd.ToDevice(scale.data());
    const double flop = 2.0 * M * N * K, bytes = (double)M * K + (double)K * N + (double)M * N + 4.0 * N;
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), {dd.GetDeviceBuffer()},
                                          de.GetDeviceBuffer(), M, N, K, sa, sb, {0}, se, Pass{}, Pass{}, CDE{});
        },
        de, (std::size_t)M * se, flop, bytes, verify, time_kernel, nrepeat);
}

int profile_gemm_perchannel_quant(int argc, char* argv[])
{
    if(argc < 9)
    {
        std::printf("arg1: tensor operation (gemm_perchannel_quant)\narg2: verification\narg3: initialization\n"
                    "arg4: print tensor value\narg5: time kernel\narg6 to 11: M, N, K, StrideA, StrideB, StrideE\n"
                    "arg12: activation (0: PassThrough; 1: Relu)\narg13: nrepeat\n");
        return 1;
    }
    const bool verify = std::atoi(argv[2]), time_kernel = std::atoi(argv[5]);
    const int init = std::atoi(argv[3]);
    const int M = std::atoi(argv[6]), N = std::atoi(argv[7]), K = std::atoi(argv[8]);
    int sa = argc > 9 ? std::atoi(argv[9]) : -1, sb = argc > 10 ? std::atoi(argv[10]) : -1,
        se = argc > 11 ? std::atoi(argv[11]) : -1;
    sa = sa < 0 ? K : sa, sb = sb < 0 ? K : sb, se = se < 0 ? N : se;
    const int act = argc > 12 ? std::atoi(argv[12]) : 1, nrepeat = argc > 13 ? std::atoi(argv[13]) : 10;
    return act ? profile_gemm_perchannel_quant_t<element_wise::Relu>(verify, init, time_kernel, M, N, K, sa, sb, se, nrepeat)
               : profile_gemm_perchannel_quant_t<Pass>(verify, init, time_kernel, M, N, K, sa, sb, se, nrepeat);
}

// E = cde(A * B, D0[, D1]) for the fp16 CDE operations with the reference's own profiler commands: Bilinear (one D
// tensor) and AddAddFastGelu (two). A D stride of 0 broadcasts one row; a negative stride stands for the dense default.
template <typename CDE, int NumD, typename AL, typename BL>
int profile_gemm_cde_l(bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sd0, int sd1,
                       int se, CDE cde, int nrepeat)
{
    using T        = half_t;
    using Ds       = std::conditional_t<NumD == 1, ck::Tuple<T>, ck::Tuple<T, T>>;
    using DeviceOp = device::DeviceGemmMultipleD<AL, BL, Row, T, T, Ds, T, Pass, Pass, CDE>;
    auto ops       = device::instance::DeviceOperationInstanceFactory<DeviceOp>::GetInstances();
    constexpr bool a_row = std::is_same_v<AL, Row>, b_row = std::is_same_v<BL, Row>;
    sa = sa < 0 ? (a_row ? K : M) : sa, sb = sb < 0 ? (b_row ? N : K) : sb, se = se < 0 ? N : se;
    sd0 = sd0 < 0 ? N : sd0, sd1 = sd1 < 0 ? N : sd1;
    std::vector<T> a((std::size_t)(a_row ? M : K) * sa), b((std::size_t)(b_row ? K : N) * sb);
    std::vector<T> d0(sd0 ? (std::size_t)M * sd0 : (std::size_t)N), d1(sd1 ? (std::size_t)M * sd1 : (std::size_t)N);
    fill(a, init, 0xC0FFEE, false);
    fill(b, init, 0xC0FFEE + 1, false);
    fill(d0, init, 0xC0FFEE + 9, false);
    fill(d1, init, 0xC0FFEE + 10, false);
    ckx::DeviceMem da(a.size() * sizeof(T)), db(b.size() * sizeof(T)), dd0(d0.size() * sizeof(T)),
        dd1(d1.size() * sizeof(T)), de((std::size_t)M * se * sizeof(T));
    da.ToDevice(a.data());
    db.ToDevice(b.data());
    dd0.ToDevice(d0.data());
    dd1.ToDevice(d1.data());
    const double flop  = 2.0 * M * N * K;
    const double bytes = sizeof(T) * ((double)M * K + (double)K * N + (double)M * N + (sd0 ? (double)M * N : (double)N) +
                                      (NumD > 1 ? (sd1 ? (double)M * N : (double)N) : 0.0));
    return run_family<T>(
        ops,
        [&](DeviceOp& op) {
            if constexpr(NumD == 1)
                return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(), {dd0.GetDeviceBuffer()},
                                              de.GetDeviceBuffer(), M, N, K, sa, sb, {sd0}, se, Pass{}, Pass{}, cde);
            else
                return op.MakeArgumentPointer(da.GetDeviceBuffer(), db.GetDeviceBuffer(),
                                              {dd0.GetDeviceBuffer(), dd1.GetDeviceBuffer()}, de.GetDeviceBuffer(), M, N,
                                              K, sa, sb, {sd0, sd1}, se, Pass{}, Pass{}, cde);
        },
        de, (std::size_t)M * se, flop, bytes, verify, time_kernel, nrepeat);
}

template <typename CDE, int NumD>
int profile_gemm_cde(int layout, bool verify, int init, bool time_kernel, int M, int N, int K, int sa, int sb, int sd0,
                     int sd1, int se, CDE cde, int nrepeat)
{
    switch(layout)
    {
    case MK_KN_MN: return profile_gemm_cde_l<CDE, NumD, Row, Row>(verify, init, time_kernel, M, N, K, sa, sb, sd0, sd1, se, cde, nrepeat);
    case MK_NK_MN: return profile_gemm_cde_l<CDE, NumD, Row, Col>(verify, init, time_kernel, M, N, K, sa, sb, sd0, sd1, se, cde, nrepeat);
    case KM_KN_MN: return profile_gemm_cde_l<CDE, NumD, Col, Row>(verify, init, time_kernel, M, N, K, sa, sb, sd0, sd1, se, cde, nrepeat);
    case KM_NK_MN: return profile_gemm_cde_l<CDE, NumD, Col, Col>(verify, init, time_kernel, M, N, K, sa, sb, sd0, sd1, se, cde, nrepeat);
    }
    std::printf("unknown matrix layout\n");
    return 1;
}

int profile_gemm_bilinear(int argc, char* argv[])
{
    if(argc < 17 || std::atoi(argv[2]) != 1)
    {
        std::printf("arg1: tensor operation (gemm_bilinear: GEMM+Bilinear)\narg2: data type (1: fp16)\n"
                    "arg3: matrix layout (0: E[m, n] = alpha * A[m, k] * B[k, n] + beta * D[m, n];\n"
                    "                     1: E[m, n] = alpha * A[m, k] * B[n, k] + beta * D[m, n];\n"
                    "                     2: E[m, n] = alpha * A[k, m] * B[k, n] + beta * D[m, n];\n"
                    "                     3: E[m, n] = alpha * A[k, m] * B[n, k] + beta * D[m, n])\n"
                    "arg4: verification (0: no; 1: yes)\narg5: initialization (0: no init; 1: integer value; 2: decimal value)\n"
                    "arg6: print tensor value (0: no; 1: yes)\narg7: time kernel (0=no, 1=yes)\n"
                    "arg8 to 14: M, N, K, StrideA, StrideB, StrideD, StrideE\narg15 to 16: alpha, beta\narg17: nrepeat\n");
        return 1;
    }
    const int layout = std::atoi(argv[3]), init = std::atoi(argv[5]);
    const bool verify = std::atoi(argv[4]), time_kernel = std::atoi(argv[7]);
    const int M = std::atoi(argv[8]), N = std::atoi(argv[9]), K = std::atoi(argv[10]);
    const int sa = std::atoi(argv[11]), sb = std::atoi(argv[12]), sd = std::atoi(argv[13]), se = std::atoi(argv[14]);
    const float alpha = (float)std::atof(argv[15]), beta = (float)std::atof(argv[16]);
    const int nrepeat = argc > 17 ? std::atoi(argv[17]) : 10;
    return profile_gemm_cde<element_wise::Bilinear, 1>(layout, verify, init, time_kernel, M, N, K, sa, sb, sd, 0, se,
                                                       element_wise::Bilinear{alpha, beta}, nrepeat);
}

int profile_gemm_add_add_fastgelu(int argc, char* argv[])
{
    if(argc < 16 || std::atoi(argv[2]) != 1)
    {
        std::printf("arg1: tensor operation (gemm_add_add_fastgelu: GEMM+Add+Add+FastGeLU)\narg2: data type (1: fp16)\n"
                    "arg3: matrix layout (0: E[m, n] = FastGeLU(A[m, k] * B[k, n] + D0[m, n] + D1[m, n]);\n"
                    "                     1: E[m, n] = FastGeLU(A[m, k] * B[n, k] + D0[m, n] + D1[m, n]);\n"
                    "                     2: E[m, n] = FastGeLU(A[k, m] * B[k, n] + D0[m, n] + D1[m, n]);\n"
                    "                     3: E[m, n] = FastGeLU(A[k, m] * B[n, k] + D0[m, n] + D1[m, n]))\n"
                    "arg4: verification (0: no; 1: yes)\narg5: initialization (0: no init; 1: integer value; 2: decimal value)\n"
                    "arg6: print tensor value (0: no; 1: yes)\narg7: time kernel (0=no, 1=yes)\n"
                    "arg8 to 15: M, N, K, StrideA, StrideB, StrideD0, StrideD1, StrideE\narg16: nrepeat\n");
        return 1;
    }
    const int layout = std::atoi(argv[3]), init = std::atoi(argv[5]);
    const bool verify = std::atoi(argv[4]), time_kernel = std::atoi(argv[7]);
    const int M = std::atoi(argv[8]), N = std::atoi(argv[9]), K = std::atoi(argv[10]);
    const int sa = std::atoi(argv[11]), sb = std::atoi(argv[12]), sd0 = std::atoi(argv[13]), sd1 = std::atoi(argv[14]),
              se = std::atoi(argv[15]);
    const int nrepeat = argc > 16 ? std::atoi(argv[16]) : 10;
    return profile_gemm_cde<element_wise::AddAddFastGelu, 2>(layout, verify, init, time_kernel, M, N, K, sa, sb, sd0,
                                                             sd1, se, element_wise::AddAddFastGelu{}, nrepeat);
}

int profile_gemm_gemm(int argc, char* argv[])
{
    if(argc < 11)
    {
        std::printf("arg1: tensor operation (batched_gemm_gemm)\narg2: verification\narg3: initialization\n"
                    "arg4: print tensor value\narg5: time kernel\narg6 to 10: M, N, K, O, Batch\nlast: nrepeat\n");
        return 1;
    }
    const bool verify = std::atoi(argv[2]), time_kernel = std::atoi(argv[5]);
    const int init = std::atoi(argv[3]);
    const int M = std::atoi(argv[6]), N = std::atoi(argv[7]), K = std::atoi(argv[8]), O = std::atoi(argv[9]),
              G = std::atoi(argv[10]);
    const int nrepeat = argc > 11 ? std::atoi(argv[11]) : 10;
    using Op = device::DeviceBatchedGemmGemm<Row, Col, Row, Row, half_t, half_t, half_t, half_t, Pass, Pass, Pass,
                                             Pass, Pass>;
    std::vector<std::unique_ptr<Op>> ops;
    for(int i = 0; i < ckx_num_instances(CKX_OP_BATCHED_GEMM_GEMM); ++i)
        ops.push_back(std::make_unique<device::DeviceBatchedGemmGemmMfma<>>(i));
    std::vector<half_t> a((std::size_t)G * M * K), b0((std::size_t)G * N * K), b1((std::size_t)G * N * O);
    if(init)
    {
        ckx::fill_uniform_f16(a, -0.5f, 0.5f, 0xC0FFEE + 4);
        ckx::fill_uniform_f16(b0, -0.5f, 0.5f, 0xC0FFEE + 5);
        ckx::fill_uniform_f16(b1, -0.5f, 0.5f, 0xC0FFEE + 6);
    }
    const std::size_t out_elems = (std::size_t)G * M * O;
    ckx::DeviceMem da(a.size() * 2), db0(b0.size() * 2), db1(b1.size() * 2), dc(out_elems * 2);
    da.ToDevice(a.data());
    db0.ToDevice(b0.data());
    db1.ToDevice(b1.data());
    const double flop  = 2.0 * G * ((double)M * N * K + (double)M * N * O);
    const double bytes = 2.0 * ((double)a.size() + b0.size() + b1.size() + out_elems);
    return run_family<half_t>(
        ops,
        [&](Op& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db0.GetDeviceBuffer(), db1.GetDeviceBuffer(),
                                          dc.GetDeviceBuffer(), M, N, K, O, G, K, K, O, O, M * K, N * K, N * O, M * O,
                                          Pass{}, Pass{}, Pass{}, Pass{}, Pass{});
        },
        dc, out_elems, flop, bytes, verify, time_kernel, nrepeat);
}

// batched_gemm_softmax_gemm <verify> <init> <log> <time> M N K O Batch [scale] [mask_out_upper_triangle] [nrepeat]
template <bool Mask>
int profile_gemm_softmax_gemm_t(bool verify, int init, bool time_kernel, int M, int N, int K, int O, int G, float scale,
                                int nrepeat)
{
    using Scale = element_wise::Scale;
    using Op = device::DeviceBatchedGemmSoftmaxGemm<Row, Col, Row, Row, half_t, half_t, half_t, half_t, Pass, Pass, Scale,
                                                    Pass, Pass, Mask>;
    std::vector<std::unique_ptr<Op>> ops;
    for(int i = 0; i < ckx_num_instances(CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM); ++i)
        ops.push_back(std::make_unique<device::DeviceBatchedGemmSoftmaxGemmMfma<Scale, Mask>>(i));
    std::vector<half_t> a((std::size_t)G * M * K), b0((std::size_t)G * N * K), b1((std::size_t)G * N * O);
    if(init)
    {
        ckx::fill_uniform_f16(a, -1.0f, 1.0f, 0xC0FFEE + 7);
        ckx::fill_uniform_f16(b0, -1.0f, 1.0f, 0xC0FFEE + 8);
        ckx::fill_uniform_f16(b1, -1.0f, 1.0f, 0xC0FFEE + 9);
    }
    const std::size_t out_elems = (std::size_t)G * M * O;
    ckx::DeviceMem da(a.size() * 2), db0(b0.size() * 2), db1(b1.size() * 2), dc(out_elems * 2);
    da.ToDevice(a.data());
    db0.ToDevice(b0.data());
    db1.ToDevice(b1.data());
    const double flop  = 2.0 * G * ((double)M * N * K + (double)M * N * O);
    const double bytes = 2.0 * ((double)a.size() + b0.size() + b1.size() + out_elems);
    return run_family<half_t>(
        ops,
        [&](Op& op) {
            return op.MakeArgumentPointer(da.GetDeviceBuffer(), db0.GetDeviceBuffer(), db1.GetDeviceBuffer(),
                                          dc.GetDeviceBuffer(), M, N, K, O, G, K, K, O, O, M * K, N * K, N * O, M * O,
                                          Pass{}, Pass{}, Scale{scale}, Pass{}, Pass{});
        },
        dc, out_elems, flop, bytes, verify, time_kernel, nrepeat);
}

int profile_gemm_softmax_gemm(int argc, char* argv[])
{
    if(argc < 11)
    {
        std::printf("arg1: tensor operation (batched_gemm_softmax_gemm)\narg2: verification\narg3: initialization\n"
                    "arg4: print tensor value\narg5: time kernel\narg6 to 10: M, N, K, O, Batch\n"
                    "arg11: score scale (default 1/sqrt(K))\narg12: mask out the upper triangle (0 | 1)\nlast: nrepeat\n");
        return 1;
    }
    const bool verify = std::atoi(argv[2]), time_kernel = std::atoi(argv[5]);
    const int init = std::atoi(argv[3]);
    const int M = std::atoi(argv[6]), N = std::atoi(argv[7]), K = std::atoi(argv[8]), O = std::atoi(argv[9]),
              G = std::atoi(argv[10]);
    const float scale = argc > 11 ? (float)std::atof(argv[11]) : 1.0f / std::sqrt((float)(K > 0 ? K : 1));
    const bool mask   = argc > 12 && std::atoi(argv[12]);
    const int nrepeat = argc > 13 ? std::atoi(argv[13]) : 10;
    return mask ? profile_gemm_softmax_gemm_t<true>(verify, init, time_kernel, M, N, K, O, G, scale, nrepeat)
                : profile_gemm_softmax_gemm_t<false>(verify, init, time_kernel, M, N, K, O, G, scale, nrepeat);
}

} // namespace

int main(int argc, char* argv[])
{
    try
    {
        if(argc >= 2 && std::strcmp(argv[1], "gemm") == 0)
            return profile_gemm(argc, argv);
        if(argc >= 2 && (std::strcmp(argv[1], "conv2d_fwd") == 0 || std::strcmp(argv[1], "conv_fwd") == 0))
            return profile_conv(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "batched_gemm_gemm") == 0)
            return profile_gemm_gemm(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "batched_gemm_softmax_gemm") == 0)
            return profile_gemm_softmax_gemm(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "convnd_fwd") == 0)
            return profile_convnd(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "conv_fwd_bias_relu") == 0)
            return profile_conv_bias_relu(argc, argv, false);
        if(argc >= 2 && std::strcmp(argv[1], "conv_fwd_bias_relu_add") == 0)
            return profile_conv_bias_relu(argc, argv, true);
        if(argc >= 2 && std::strcmp(argv[1], "batched_gemm") == 0)
            return profile_batched_gemm(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "gemm_splitk") == 0)
            return profile_gemm_splitk(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "gemm_perchannel_quant") == 0)
            return profile_gemm_perchannel_quant(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "gemm_bias_relu") == 0)
            return profile_gemm_bias_relu(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "gemm_bilinear") == 0)
            return profile_gemm_bilinear(argc, argv);
        if(argc >= 2 && std::strcmp(argv[1], "gemm_add_add_fastgelu") == 0)
            return profile_gemm_add_add_fastgelu(argc, argv);
        std::printf("arg1: tensor operation (gemm: GEMM\n"
                    "                        conv2d_fwd: NHWC/KYXC/NHWK forward convolution\n"
                    "                        batched_gemm_gemm: batched fused GEMM+GEMM\n"
                    "                        batched_gemm_softmax_gemm: batched fused GEMM+Softmax+GEMM\n"
                    "                        convnd_fwd: forward convolution, 1 / 2 / 3 spatial dimensions, channels last\n"
                    "                        conv_fwd_bias_relu: ForwardConvolution+Bias+ReLU\n"
                    "                        conv_fwd_bias_relu_add: ForwardConvolution+Bias+ReLU+Add\n"
                    "                        batched_gemm: Batched GEMM\n"
                    "                        gemm_splitk: Split-K GEMM\n"
                    "                        gemm_bias_relu: GEMM+Bias+ReLU)\n");
        return 1;
    }
    catch(const std::exception& e)
    {
        std::cerr << e.what() << std::endl;
        return 2;
    }
}
