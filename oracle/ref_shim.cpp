// C-ABI shim around the reference's OWN host operators, compiled from the
// sources where they lie under /root/reference (never copied). TEST
// INFRASTRUCTURE ONLY: validates oracle/ck_oracle.cpp and can serve as the
// benchmark's cpu_baseline. Built by oracle/Makefile into oracle/_ref/.
//
// Instantiates, exactly as the reference's examples/tests/profiler do:
//   ReferenceGemm<int8,int8,int8,float,Pass,Pass,RequantReluRequant>  (example 14, :103-109)
//   ReferenceGemm<int8,int8,int8,int32,Pass,Pass,Pass>                 (profile_gemm.cpp int8)
//   ReferenceGemm<half,half,half,float,Pass,Pass,Pass>                 (example 01 fp16)
//   ReferenceConvFwd<T,T,T,Pass,Pass,Pass,2> for float / half / int8
//   ReferenceBatchedGemm<half,half,half,Pass,Pass,Pass>
//   ReferenceBatchedGemm<half,half,float,Pass,Pass,Scale> -> ReferenceSoftmax<float,half,float> ->
//   ReferenceBatchedGemm<half,half,half,...>: the pieces of the fused GEMM + softmax + GEMM check
//
// RequantReluRequant lives inside the example's translation unit
// (example/14_.../gemm_xdl_requant_relu_requant_int8.cpp:21-39), which also pulls
// in the device-side headers; those do not compile with this ROCm release
// (get_id.hpp's constexpr warpSize), so the five-line functor is restated here
// and handed to the reference's own ReferenceGemm template. The rounded variant
// has no counterpart in the reference at all.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "ck/utility/magic_division.hpp"
#include "ck/tensor_operation/gpu/element/element_wise_operation.hpp"
#include "ck/library/host_tensor/host_tensor.hpp"
#include "ck/library/utility/conv_util.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_gemm.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_conv_fwd.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_batched_gemm.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_softmax.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_conv_fwd_bias_activation.hpp"
#include "ck/library/reference_tensor_operation/cpu/reference_conv_fwd_bias_activation_add.hpp"

namespace {

using PassThrough = ck::tensor_operation::element_wise::PassThrough;

struct RequantReluRequant
{
    RequantReluRequant(float sg, float sr) : sg_(sg), sr_(sr) {}
    void operator()(float& y, const float& x) const
    {
        float g = sg_ * x;
        float r = g > 0 ? g : 0;
        float q = sr_ * r;
        y       = q > 127 ? 127 : q < -128 ? -128 : q;
    }
    float sg_, sr_;
};

using ReferenceGemmInstance = ck::tensor_operation::host::
    ReferenceGemm<int8_t, int8_t, int8_t, float, PassThrough, PassThrough, RequantReluRequant>;

struct RequantRoundReluRequantRound
{
    RequantRoundReluRequantRound(float sg, float sr) : sg_(sg), sr_(sr) {}
    void operator()(float& y, const float& x) const
    {
        float t = std::nearbyint(sg_ * x);
        t       = t > 127 ? 127 : (t < -128 ? -128 : t);
        float r = t > 0 ? t : 0;
        float u = std::nearbyint(sr_ * r);
        y       = u > 127 ? 127 : (u < -128 ? -128 : u);
    }
    float sg_, sr_;
};

template <typename T>
Tensor<T> make_tensor(std::vector<std::size_t> lens, std::vector<std::size_t> strides, const T* src)
{
    Tensor<T> t(HostTensorDescriptor(lens, strides));
    if(src)
        std::memcpy(t.mData.data(), src, t.mData.size() * sizeof(T));
    return t;
}

template <typename Ref, typename TA, typename TC, typename COp>
void run_gemm(const TA* a, const TA* b, TC* c, int M, int N, int K, long sa_m, long sa_k, long sb_k,
              long sb_n, long sc_m, long sc_n, COp cop)
{
    using sz = std::size_t;
    auto ta  = make_tensor<TA>({(sz)M, (sz)K}, {(sz)sa_m, (sz)sa_k}, a);
    auto tb  = make_tensor<TA>({(sz)K, (sz)N}, {(sz)sb_k, (sz)sb_n}, b);
    auto tc  = make_tensor<TC>({(sz)M, (sz)N}, {(sz)sc_m, (sz)sc_n}, c);
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ta, tb, tc, PassThrough{}, PassThrough{}, cop);
    inv.Run(arg);
    std::memcpy(c, tc.mData.data(), tc.mData.size() * sizeof(TC));
}

template <typename T>
void run_conv(const T* in, const T* wei, T* out, int N, int K, int C, int Hi, int Wi, int Y, int X,
              int Ho, int Wo, int sH, int sW, int dH, int dW, int pH, int pW)
{
    using sz = std::size_t;
    // logical N,C,H,W with NHWC strides (conv_util.hpp:209-215)
    auto ti = make_tensor<T>({(sz)N, (sz)C, (sz)Hi, (sz)Wi},
                             {(sz)C * Hi * Wi, 1, (sz)Wi * C, (sz)C}, in);
    auto tw = make_tensor<T>({(sz)K, (sz)C, (sz)Y, (sz)X}, {(sz)C * Y * X, 1, (sz)X * C, (sz)C}, wei);
    auto to = make_tensor<T>({(sz)N, (sz)K, (sz)Ho, (sz)Wo},
                             {(sz)K * Ho * Wo, 1, (sz)Wo * K, (sz)K}, (const T*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceConvFwd<T, T, T, PassThrough, PassThrough, PassThrough, 2>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ti, tw, to, {sH, sW}, {dH, dW}, {pH, pW}, {pH, pW}, PassThrough{},
                                PassThrough{}, PassThrough{});
    inv.Run(arg);
    std::memcpy(out, to.mData.data(), to.mData.size() * sizeof(T));
}

// NumDimSpatial = ND: tensors addressed logically N,C,(D,)(H,)W with the channels-last strides of
// conv_util.hpp:195-236 (NWC / NHWC / NDHWC and the matching weight / output layouts)
template <typename T, int ND>
void run_convnd(const T* in, const T* wei, T* out, int N, int K, int C, const int* in_len, const int* filt,
                const int* out_len, const int* stride, const int* dil, const int* pad)
{
    using sz = std::size_t;
    auto desc = [](sz n, sz c, const int* len) {
        std::vector<sz> lens{n, c}, strides(2 + ND);
        sz px = 1;
        for(int i = 0; i < ND; ++i)
        {
            lens.push_back((sz)len[i]);
            px *= (sz)len[i];
        }
        strides[0] = c * px;
        strides[1] = 1;
        sz run     = c;
        for(int i = ND - 1; i >= 0; --i)
        {
            strides[2 + i] = run;
            run *= (sz)len[i];
        }
        return std::make_pair(lens, strides);
    };
    auto di = desc((sz)N, (sz)C, in_len), dw = desc((sz)K, (sz)C, filt), dq = desc((sz)N, (sz)K, out_len);
    auto ti = make_tensor<T>(di.first, di.second, in);
    auto tw = make_tensor<T>(dw.first, dw.second, wei);
    auto to = make_tensor<T>(dq.first, dq.second, (const T*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceConvFwd<T, T, T, PassThrough, PassThrough, PassThrough, ND>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    std::vector<ck::index_t> st(stride, stride + ND), dl(dil, dil + ND), pd(pad, pad + ND);
    auto arg = ref.MakeArgument(ti, tw, to, st, dl, pd, pd, PassThrough{}, PassThrough{}, PassThrough{});
    inv.Run(arg);
    std::memcpy(out, to.mData.data(), to.mData.size() * sizeof(T));
}

template <typename T>
void run_convnd_dispatch(int ndim, const T* in, const T* wei, T* out, int N, int K, int C, const int* in_len,
                         const int* filt, const int* out_len, const int* stride, const int* dil, const int* pad)
{
    if(ndim == 1)
        run_convnd<T, 1>(in, wei, out, N, K, C, in_len, filt, out_len, stride, dil, pad);
    else if(ndim == 2)
        run_convnd<T, 2>(in, wei, out, N, K, C, in_len, filt, out_len, stride, dil, pad);
    else
        run_convnd<T, 3>(in, wei, out, N, K, C, in_len, filt, out_len, stride, dil, pad);
}

} // namespace

extern "C" {

// epi: 1 = example-14 functor, 2 = rounded variant
void ckref_gemm_i8_requant(const int8_t* a, const int8_t* b, int8_t* c, int M, int N, int K, long sa_m,
                           long sa_k, long sb_k, long sb_n, long sc_m, long sc_n, int epi,
                           float scale_gemm, float scale_relu)
{
    if(epi == 1)
        run_gemm<ReferenceGemmInstance, int8_t, int8_t>(a, b, c, M, N, K, sa_m, sa_k, sb_k, sb_n, sc_m,
                                                        sc_n, RequantReluRequant{scale_gemm, scale_relu});
    else
        run_gemm<ck::tensor_operation::host::ReferenceGemm<int8_t, int8_t, int8_t, float, PassThrough,
                                                           PassThrough, RequantRoundReluRequantRound>,
                 int8_t, int8_t>(a, b, c, M, N, K, sa_m, sa_k, sb_k, sb_n, sc_m, sc_n,
                                 RequantRoundReluRequantRound{scale_gemm, scale_relu});
}

void ckref_gemm_i8(const int8_t* a, const int8_t* b, int8_t* c, int M, int N, int K, long sa_m,
                   long sa_k, long sb_k, long sb_n, long sc_m, long sc_n)
{
    run_gemm<ck::tensor_operation::host::ReferenceGemm<int8_t, int8_t, int8_t, int32_t, PassThrough,
                                                       PassThrough, PassThrough>,
             int8_t, int8_t>(a, b, c, M, N, K, sa_m, sa_k, sb_k, sb_n, sc_m, sc_n, PassThrough{});
}

void ckref_gemm_f16(const uint16_t* a, const uint16_t* b, uint16_t* c, int M, int N, int K, long sa_m,
                    long sa_k, long sb_k, long sb_n, long sc_m, long sc_n)
{
    using H = ck::half_t;
    run_gemm<ck::tensor_operation::host::ReferenceGemm<H, H, H, float, PassThrough, PassThrough,
                                                       PassThrough>,
             H, H>((const H*)a, (const H*)b, (H*)c, M, N, K, sa_m, sa_k, sb_k, sb_n, sc_m, sc_n,
                   PassThrough{});
}

void ckref_conv2d_fwd_f32(const float* in, const float* wei, float* out, int N, int K, int C, int Hi,
                          int Wi, int Y, int X, int Ho, int Wo, int sH, int sW, int dH, int dW, int pH,
                          int pW)
{
    run_conv<float>(in, wei, out, N, K, C, Hi, Wi, Y, X, Ho, Wo, sH, sW, dH, dW, pH, pW);
}

void ckref_conv2d_fwd_f16(const uint16_t* in, const uint16_t* wei, uint16_t* out, int N, int K, int C,
                          int Hi, int Wi, int Y, int X, int Ho, int Wo, int sH, int sW, int dH, int dW,
                          int pH, int pW)
{
    using H = ck::half_t;
    run_conv<H>((const H*)in, (const H*)wei, (H*)out, N, K, C, Hi, Wi, Y, X, Ho, Wo, sH, sW, dH, dW, pH,
                pW);
}

void ckref_conv2d_fwd_i8(const int8_t* in, const int8_t* wei, int8_t* out, int N, int K, int C, int Hi,
                         int Wi, int Y, int X, int Ho, int Wo, int sH, int sW, int dH, int dW, int pH,
                         int pW)
{
    run_conv<int8_t>(in, wei, out, N, K, C, Hi, Wi, Y, X, Ho, Wo, sH, sW, dH, dW, pH, pW);
}

// ndim spatial dimensions, the first ndim entries of every array are used (slowest dimension first); symmetric pads
void ckref_convnd_fwd_f32(int ndim, const float* in, const float* wei, float* out, int N, int K, int C,
                          const int* in_len, const int* filt, const int* out_len, const int* stride, const int* dil,
                          const int* pad)
{
    run_convnd_dispatch<float>(ndim, in, wei, out, N, K, C, in_len, filt, out_len, stride, dil, pad);
}

void ckref_convnd_fwd_f16(int ndim, const uint16_t* in, const uint16_t* wei, uint16_t* out, int N, int K, int C,
                          const int* in_len, const int* filt, const int* out_len, const int* stride, const int* dil,
                          const int* pad)
{
    using H = ck::half_t;
    run_convnd_dispatch<H>(ndim, (const H*)in, (const H*)wei, (H*)out, N, K, C, in_len, filt, out_len, stride, dil,
                           pad);
}

void ckref_convnd_fwd_i8(int ndim, const int8_t* in, const int8_t* wei, int8_t* out, int N, int K, int C,
                         const int* in_len, const int* filt, const int* out_len, const int* stride, const int* dil,
                         const int* pad)
{
    run_convnd_dispatch<int8_t>(ndim, in, wei, out, N, K, C, in_len, filt, out_len, stride, dil, pad);
}

void ckref_batched_gemm_f16(const uint16_t* a, const uint16_t* b, uint16_t* c, int G, int M, int N,
                            int K, long sa_g, long sa_m, long sa_k, long sb_g, long sb_k, long sb_n,
                            long sc_g, long sc_m, long sc_n)
{
    using H  = ck::half_t;
    using sz = std::size_t;
    auto ta  = make_tensor<H>({(sz)G, (sz)M, (sz)K}, {(sz)sa_g, (sz)sa_m, (sz)sa_k}, (const H*)a);
    auto tb  = make_tensor<H>({(sz)G, (sz)K, (sz)N}, {(sz)sb_g, (sz)sb_k, (sz)sb_n}, (const H*)b);
    auto tc  = make_tensor<H>({(sz)G, (sz)M, (sz)N}, {(sz)sc_g, (sz)sc_m, (sz)sc_n}, (const H*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceBatchedGemm<H, H, H, PassThrough, PassThrough, PassThrough>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ta, tb, tc, PassThrough{}, PassThrough{}, PassThrough{});
    inv.Run(arg);
    std::memcpy(c, tc.mData.data(), tc.mData.size() * sizeof(H));
}

// scores = Scale(A * B0) in fp32 (the reference's ReferenceBatchedGemm and element_wise::Scale), optional
// upper-triangle mask, the reference's ReferenceSoftmax over n (float in, half out, alpha 1, beta 0),
// then the reference's ReferenceBatchedGemm with B1
void ckref_batched_gemm_softmax_gemm_f16(const uint16_t* a, const uint16_t* b0, const uint16_t* b1, uint16_t* c,
                                         int G, int M, int N, int K, int O, long sa_g, long sa_m, long sa_k,
                                         long sb0_g, long sb0_k, long sb0_n, long sb1_g, long sb1_n, long sb1_o,
                                         float scale, int mask_upper)
{
    using H     = ck::half_t;
    using sz    = std::size_t;
    using Scale = ck::tensor_operation::element_wise::Scale;
    auto ta  = make_tensor<H>({(sz)G, (sz)M, (sz)K}, {(sz)sa_g, (sz)sa_m, (sz)sa_k}, (const H*)a);
    auto tb0 = make_tensor<H>({(sz)G, (sz)K, (sz)N}, {(sz)sb0_g, (sz)sb0_k, (sz)sb0_n}, (const H*)b0);
    auto tb1 = make_tensor<H>({(sz)G, (sz)N, (sz)O}, {(sz)sb1_g, (sz)sb1_n, (sz)sb1_o}, (const H*)b1);
    Tensor<float> acc0(HostTensorDescriptor(std::vector<sz>{(sz)G, (sz)M, (sz)N}));
    Tensor<H> prob(HostTensorDescriptor(std::vector<sz>{(sz)G, (sz)M, (sz)N}));
    Tensor<H> tc(HostTensorDescriptor(std::vector<sz>{(sz)G, (sz)M, (sz)O}));
    {
        using Ref = ck::tensor_operation::host::ReferenceBatchedGemm<H, H, float, PassThrough, PassThrough, Scale>;
        Ref ref;
        auto inv = ref.MakeInvoker();
        auto arg = ref.MakeArgument(ta, tb0, acc0, PassThrough{}, PassThrough{}, Scale{scale});
        inv.Run(arg);
    }
    if(mask_upper)
        acc0.ForEach([&](auto& self, auto idx) {
            if(idx[2] > idx[1])
                self(idx) = -std::numeric_limits<float>::infinity();
        });
    {
        using Ref = ck::tensor_operation::host::ReferenceSoftmax<float, H, float>;
        Ref ref;
        auto inv = ref.MakeInvoker();
        auto arg = ref.MakeArgument(acc0, prob, 1.0f, 0.0f, {2});
        inv.Run(arg);
    }
    {
        using Ref = ck::tensor_operation::host::ReferenceBatchedGemm<H, H, H, PassThrough, PassThrough, PassThrough>;
        Ref ref;
        auto inv = ref.MakeInvoker();
        auto arg = ref.MakeArgument(prob, tb1, tc, PassThrough{}, PassThrough{}, PassThrough{});
        inv.Run(arg);
    }
    std::memcpy(c, tc.mData.data(), tc.mData.size() * sizeof(H));
}

// ReferenceConvFwd_Bias_Activation<half,half,half,Pass,Pass,AddRelu> (example 06) and
// ReferenceConvFwd_Bias_Activation_Add<..., AddReluAdd> (example 07); resi == null selects the former
void ckref_conv2d_fwd_bias_relu_f16(const uint16_t* in, const uint16_t* wei, const uint16_t* bias,
                                    const uint16_t* resi, uint16_t* out, int N, int K, int C, int Hi, int Wi,
                                    int Y, int X, int Ho, int Wo, int sH, int sW, int dH, int dW, int pH,
                                    int pW)
{
    using T  = ck::half_t;
    using sz = std::size_t;
    auto ti  = make_tensor<T>({(sz)N, (sz)C, (sz)Hi, (sz)Wi}, {(sz)C * Hi * Wi, 1, (sz)Wi * C, (sz)C},
                             reinterpret_cast<const T*>(in));
    auto tw  = make_tensor<T>({(sz)K, (sz)C, (sz)Y, (sz)X}, {(sz)C * Y * X, 1, (sz)X * C, (sz)C},
                             reinterpret_cast<const T*>(wei));
    auto to  = make_tensor<T>({(sz)N, (sz)K, (sz)Ho, (sz)Wo}, {(sz)K * Ho * Wo, 1, (sz)Wo * K, (sz)K},
                             (const T*)nullptr);
    auto tb  = make_tensor<T>({(sz)K}, {1}, reinterpret_cast<const T*>(bias));
    if(resi)
    {
        auto tr = make_tensor<T>({(sz)N, (sz)K, (sz)Ho, (sz)Wo}, {(sz)K * Ho * Wo, 1, (sz)Wo * K, (sz)K},
                                 reinterpret_cast<const T*>(resi));
        using Op  = ck::tensor_operation::element_wise::AddReluAdd;
        using Ref = ck::tensor_operation::host::ReferenceConvFwd_Bias_Activation_Add<T, T, T, PassThrough,
                                                                                     PassThrough, Op>;
        Ref ref;
        auto inv = ref.MakeInvoker();
        auto arg = ref.MakeArgument(ti, tw, to, tb, tr, {sH, sW}, {dH, dW}, {pH, pW}, {pH, pW}, PassThrough{},
                                    PassThrough{}, Op{});
        inv.Run(arg);
    }
    else
    {
        using Op  = ck::tensor_operation::element_wise::AddRelu;
        using Ref = ck::tensor_operation::host::ReferenceConvFwd_Bias_Activation<T, T, T, PassThrough,
                                                                                 PassThrough, Op>;
        Ref ref;
        auto inv = ref.MakeInvoker();
        auto arg = ref.MakeArgument(ti, tw, to, tb, {sH, sW}, {dH, dW}, {pH, pW}, {pH, pW}, PassThrough{},
                                    PassThrough{}, Op{});
        inv.Run(arg);
    }
    std::memcpy(out, to.mData.data(), to.mData.size() * sizeof(T));
}

// ReferenceGemm<bhalf_t, bhalf_t, bhalf_t, float, Pass, Pass, Pass> (the reference's bf16 GEMM check)
void ckref_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c, int M, int N, int K, long sa_m,
                     long sa_k, long sb_k, long sb_n, long sc_m, long sc_n)
{
    using Ref = ck::tensor_operation::host::ReferenceGemm<ck::bhalf_t, ck::bhalf_t, ck::bhalf_t, float, PassThrough,
                                                          PassThrough, PassThrough>;
    run_gemm<Ref, ck::bhalf_t, ck::bhalf_t>(a, b, c, M, N, K, sa_m, sa_k, sb_k, sb_n, sc_m, sc_n, PassThrough{});
}

uint16_t ckref_float_to_bf16(float x) { return ck::type_convert<ck::bhalf_t>(x); }

// example 03's verification: ReferenceGemm<half,half,float,float,...> then AddRelu on half_t
void ckref_gemm_f16_add_relu(const uint16_t* a, const uint16_t* b, const uint16_t* d, uint16_t* e, int M, int N,
                             int K, long sa_m, long sa_k, long sb_k, long sb_n, long sd_m, long sd_n)
{
    using T  = ck::half_t;
    using sz = std::size_t;
    auto ta  = make_tensor<T>({(sz)M, (sz)K}, {(sz)sa_m, (sz)sa_k}, reinterpret_cast<const T*>(a));
    auto tb  = make_tensor<T>({(sz)K, (sz)N}, {(sz)sb_k, (sz)sb_n}, reinterpret_cast<const T*>(b));
    auto tc  = make_tensor<float>({(sz)M, (sz)N}, {(sz)N, 1}, (const float*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceGemm<T, T, float, float, PassThrough, PassThrough, PassThrough>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ta, tb, tc, PassThrough{}, PassThrough{}, PassThrough{});
    inv.Run(arg);
    const T* dd = reinterpret_cast<const T*>(d);
    T* ee       = reinterpret_cast<T*>(e);
    ck::tensor_operation::element_wise::AddRelu op;
    for(int m = 0; m < M; ++m)
        for(int n = 0; n < N; ++n)
        {
            const T c = ck::type_convert<T>(tc(m, n));
            op(ee[(sz)m * N + n], c, dd[(sz)m * sd_m + (sz)n * sd_n]);
        }
}

// example 02's verification: ReferenceGemm<half,half,float,float,...> then the reference's own Bilinear functor
// (binary_element_wise_operation.hpp:93-116) on (half_t&, const float&, const half_t&)
void ckref_gemm_f16_bilinear(const uint16_t* a, const uint16_t* b, const uint16_t* d, uint16_t* e, int M, int N,
                             int K, long sa_m, long sa_k, long sb_k, long sb_n, long sd_m, long sd_n, float alpha,
                             float beta)
{
    using T  = ck::half_t;
    using sz = std::size_t;
    auto ta  = make_tensor<T>({(sz)M, (sz)K}, {(sz)sa_m, (sz)sa_k}, reinterpret_cast<const T*>(a));
    auto tb  = make_tensor<T>({(sz)K, (sz)N}, {(sz)sb_k, (sz)sb_n}, reinterpret_cast<const T*>(b));
    auto tc  = make_tensor<float>({(sz)M, (sz)N}, {(sz)N, 1}, (const float*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceGemm<T, T, float, float, PassThrough, PassThrough, PassThrough>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ta, tb, tc, PassThrough{}, PassThrough{}, PassThrough{});
    inv.Run(arg);
    const T* dd = reinterpret_cast<const T*>(d);
    T* ee       = reinterpret_cast<T*>(e);
    ck::tensor_operation::element_wise::Bilinear op{alpha, beta};
    for(int m = 0; m < M; ++m)
        for(int n = 0; n < N; ++n)
            op(ee[(sz)m * N + n], tc(m, n), dd[(sz)m * sd_m + (sz)n * sd_n]);
}

// example 04's verification: ReferenceGemm into fp32, then the reference's own AddAddFastGelu functor
// (element_wise_operation.hpp:113-140) on (half_t&, const float&, const half_t&, const half_t&)
void ckref_gemm_f16_add_add_fastgelu(const uint16_t* a, const uint16_t* b, const uint16_t* d0, const uint16_t* d1,
                                     uint16_t* e, int M, int N, int K, long sa_m, long sa_k, long sb_k, long sb_n,
                                     long sd0_m, long sd0_n, long sd1_m, long sd1_n)
{
    using T  = ck::half_t;
    using sz = std::size_t;
    auto ta  = make_tensor<T>({(sz)M, (sz)K}, {(sz)sa_m, (sz)sa_k}, reinterpret_cast<const T*>(a));
    auto tb  = make_tensor<T>({(sz)K, (sz)N}, {(sz)sb_k, (sz)sb_n}, reinterpret_cast<const T*>(b));
    auto tc  = make_tensor<float>({(sz)M, (sz)N}, {(sz)N, 1}, (const float*)nullptr);
    using Ref =
        ck::tensor_operation::host::ReferenceGemm<T, T, float, float, PassThrough, PassThrough, PassThrough>;
    Ref ref;
    auto inv = ref.MakeInvoker();
    auto arg = ref.MakeArgument(ta, tb, tc, PassThrough{}, PassThrough{}, PassThrough{});
    inv.Run(arg);
    const T* p0 = reinterpret_cast<const T*>(d0);
    const T* p1 = reinterpret_cast<const T*>(d1);
    T* ee       = reinterpret_cast<T*>(e);
    ck::tensor_operation::element_wise::AddAddFastGelu op;
    for(int m = 0; m < M; ++m)
        for(int n = 0; n < N; ++n)
            op(ee[(sz)m * N + n], tc(m, n), p0[(sz)m * sd0_m + (sz)n * sd0_n], p1[(sz)m * sd1_m + (sz)n * sd1_n]);
}

float ckref_fast_gelu(float x)
{
    float y;
    ck::tensor_operation::element_wise::FastGelu{}(y, x);
    return y;
}

int ckref_conv_out_len(int in_len, int filter_len, int stride, int dilation, int pad_left, int pad_right)
{
    ck::utils::conv::ConvParams p;
    p.num_dim_spatial_        = 1;
    p.filter_spatial_lengths_ = {filter_len};
    p.input_spatial_lengths_  = {in_len};
    p.conv_filter_strides_    = {stride};
    p.conv_filter_dilations_  = {dilation};
    p.input_left_pads_        = {pad_left};
    p.input_right_pads_       = {pad_right};
    return p.GetOutputSpatialLengths()[0];
}

void ckref_magic_division_params(uint32_t divisor, uint32_t* multiplier, uint32_t* shift)
{
    auto t      = ck::MagicDivision::CalculateMagicNumbers(divisor);
    *multiplier = t[ck::Number<0>{}];
    *shift      = t[ck::Number<1>{}];
}

uint32_t ckref_magic_division_divide(uint32_t dividend, uint32_t multiplier, uint32_t shift)
{
    return ck::MagicDivision::DoMagicDivision(dividend, multiplier, shift);
}

} // extern "C"
