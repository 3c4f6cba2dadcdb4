// Host-side operator surface over the C ABI (include/ckx.h), carrying Composable Kernel's
// own names so that code written against the reference's device operators compiles against
// this header instead:
//
//   ck::StreamConfig                                  include/ck/stream_config.hpp:9-13
//   ck::tensor_operation::device::BaseArgument/BaseInvoker/BaseOperator
//                                                     .../gpu/device/device_base.hpp:14-57
//   ...::device::DeviceGemm<...>                      .../gpu/device/device_gemm.hpp:24-41
//   ...::device::DeviceConvFwd<...>                   .../gpu/device/device_conv_fwd.hpp:18-39
//   ...::device::DeviceBatchedGemmGemm<...>           upstream device_batched_gemm_gemm.hpp:15-56
//   ...::device::instance::DeviceOperationInstanceFactory<DeviceOp>::GetInstances()
//                                  library/.../tensor_operation_instance/gpu/gemm.hpp:233-379
//   element_wise::PassThrough                         .../gpu/element/unary_element_wise_operation.hpp:13-25
//
// The kernels are precompiled in libckx.so; an element-wise functor is therefore not inlined
// into a kernel but MAPPED to one of the library's fused epilogues through
// ckx::EpilogueOf<Functor> (specialise it for your own functor type; a functor with public
// members scaleGemm_ and scaleRelu_, like example 14's RequantReluRequant, is recognised
// automatically). Unsupported problems make IsSupportedArgument() return false and Run()
// throw std::runtime_error, as the reference does (device_gemm_xdl_cshuffle.hpp:475-481).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <array>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "ckx.h"

namespace ck {

using index_t      = int32_t;
using long_index_t = int64_t;
using half_t       = _Float16;
using bhalf_t      = unsigned short; // bfloat16 bit pattern (include/ck/utility/data_type.hpp:10)

struct StreamConfig
{
    hipStream_t stream_id_ = nullptr;
    bool time_kernel_      = false;
    int nrepeat_           = 10; // launch_and_time_kernel: 1 warm-up + 10 timed launches
    int nwarmup_           = 1;
};

namespace tensor_layout {
namespace gemm {
struct RowMajor
{
    static constexpr int code = CKX_ROW_MAJOR;
};
struct ColumnMajor
{
    static constexpr int code = CKX_COL_MAJOR;
};
} // namespace gemm
namespace convolution {
struct NHWC
{
};
struct KYXC
{
};
struct NHWK
{
};
} // namespace convolution
} // namespace tensor_layout

namespace tensor_operation {
namespace element_wise {

struct PassThrough
{
    template <typename Y, typename X>
    void operator()(Y& y, const X& x) const
    {
        y = static_cast<Y>(x);
    }
};

// y = scale * x (unary_element_wise_operation.hpp:27-41)
struct Scale
{
    Scale(float scale = 1.0f) : scale_(scale) {}
    void operator()(float& y, const float& x) const { y = scale_ * x; }
    float scale_;
};

// y = clamp(scaleRelu * relu(scaleGemm * x), -128, 127); the int8 cast truncates
// (example/14_gemm_xdl_requant_relu_requant/gemm_xdl_requant_relu_requant_int8.cpp:21-39)
struct RequantReluRequant
{
    RequantReluRequant(float scaleGemm, float scaleRelu) : scaleGemm_(scaleGemm), scaleRelu_(scaleRelu) {}
    void operator()(float& y, const float& x) const
    {
        float g = scaleGemm_ * x;
        float r = g > 0 ? g : 0;
        float q = scaleRelu_ * r;
        y       = q > 127 ? 127 : q < -128 ? -128 : q;
    }
    float scaleGemm_, scaleRelu_;
};

// y = sat8(rint(scaleRelu * relu(sat8(rint(scaleGemm * x))))), rint = round-half-to-even
struct RequantRoundReluRequantRound
{
    RequantRoundReluRequantRound(float scaleGemm, float scaleRelu) : scaleGemm_(scaleGemm), scaleRelu_(scaleRelu)
    {
    }
    float scaleGemm_, scaleRelu_;
};

// y = relu(x0 + x1) (binary_element_wise_operation.hpp:118-146). On the conv operators x0 is the
// fp32 accumulator; as the CDE operation of DeviceGemmMultipleD x0 is C already rounded to fp16.
struct AddRelu
{
    template <typename Y, typename X0, typename X1>
    void operator()(Y& y, const X0& x0, const X1& x1) const
    {
        const Y a = static_cast<Y>(x0 + x1);
        y         = a > Y(0) ? a : Y(0);
    }
};

// y = relu(x0 + x1) + x2 in fp32 (element_wise_operation.hpp:46-81)
struct AddReluAdd
{
    template <typename Y, typename X0, typename X1, typename X2>
    void operator()(Y& y, const X0& x0, const X1& x1, const X2& x2) const
    {
        const float a = static_cast<float>(x0) + static_cast<float>(x1);
        y             = static_cast<Y>((a > 0 ? a : 0) + static_cast<float>(x2));
    }
};

// y = alpha * x0 + beta * x1 in fp32, x0 the fp32 accumulator (binary_element_wise_operation.hpp:93-116)
struct Bilinear
{
    Bilinear(float alpha = 1.f, float beta = 1.f) : alpha_(alpha), beta_(beta) {}
    template <typename Y, typename X0, typename X1>
    void operator()(Y& y, const X0& x0, const X1& x1) const
    {
        y = static_cast<Y>(alpha_ * static_cast<float>(x0) + beta_ * static_cast<float>(x1));
    }
    float alpha_, beta_;
};

// y = x * cdf, the logistic form of the tanh GELU approximation (unary_element_wise_operation.hpp:121-135)
struct FastGelu
{
    void operator()(float& y, const float& x) const
    {
        const float u   = 2.f * x * (0.035677f * x * x + 0.797885f);
        const float emu = std::exp(-u);
        y               = x * (0.5f + 0.5f * (2.f / (1.f + emu) - 1.f));
    }
};

// e = fast_gelu(c + d0 + d1) on the fp32 accumulator c (element_wise_operation.hpp:113-140)
struct AddAddFastGelu
{
    template <typename E, typename C, typename D0, typename D1>
    void operator()(E& e, const C& c, const D0& d0, const D1& d1) const
    {
        float y;
        FastGelu{}(y, static_cast<float>(c) + static_cast<float>(d0) + static_cast<float>(d1));
        e = static_cast<E>(y);
    }
};

// y = x > 0 ? x : 0 (unary_element_wise_operation.hpp, Relu)
struct Relu
{
    template <typename T>
    void operator()(T& y, const T& x) const
    {
        y = x > T(0) ? x : T(0);
    }
};

// Per-channel requantisation of an int32 accumulator: upstream Composable Kernel's Activation_Mul2_Clamp<Activation>
// (ck/tensor_operation/gpu/element/quantization_operation.hpp as shipped with ROCm; newer than the reference
// snapshot). requantScale is the D operand: one fp32 value per output column / output channel.
//   y = float(x); y = activation(y); y = clamp(requantScale * y, -128, 127); e = int8(y)  (toward zero)
template <typename Activation>
struct Activation_Mul2_Clamp
{
    Activation_Mul2_Clamp(Activation activationOp = {}) : activationOp_(activationOp) {}
    void operator()(int8_t& y, const int32_t& x, const float& requantScale) const
    {
        float f = static_cast<float>(x);
        activationOp_(f, f);
        f = requantScale * f;
        f = f < -128.f ? -128.f : f > 127.f ? 127.f : f;
        y = static_cast<int8_t>(f);
    }
    Activation activationOp_;
};

} // namespace element_wise
} // namespace tensor_operation

// ck::Tuple as a type list (include/ck/utility/tuple.hpp): only Size() is needed here
template <typename... Ts>
struct Tuple
{
    static constexpr index_t Size() { return sizeof...(Ts); }
};
} // namespace ck

namespace ckx {

// Functor type -> fused epilogue of the library.
template <typename Op, typename = void>
struct EpilogueOf; // not defined: an unknown functor is a compile error, not a silent PassThrough

template <>
struct EpilogueOf<ck::tensor_operation::element_wise::PassThrough>
{
    static constexpr int kind = CKX_EPI_PASSTHROUGH;
    static float scale_gemm(const ck::tensor_operation::element_wise::PassThrough&) { return 1.f; }
    static float scale_relu(const ck::tensor_operation::element_wise::PassThrough&) { return 1.f; }
};

template <>
struct EpilogueOf<ck::tensor_operation::element_wise::RequantRoundReluRequantRound>
{
    using Op                  = ck::tensor_operation::element_wise::RequantRoundReluRequantRound;
    static constexpr int kind = CKX_EPI_REQUANT_RND;
    static float scale_gemm(const Op& o) { return o.scaleGemm_; }
    static float scale_relu(const Op& o) { return o.scaleRelu_; }
};

// any functor shaped like example 14's RequantReluRequant
template <typename Op>
struct EpilogueOf<Op,
                  std::enable_if_t<!std::is_same_v<Op, ck::tensor_operation::element_wise::RequantRoundReluRequantRound> &&
                                   std::is_same_v<decltype(std::declval<Op>().scaleGemm_), float> &&
                                   std::is_same_v<decltype(std::declval<Op>().scaleRelu_), float>>>
{
    static constexpr int kind = CKX_EPI_REQUANT_CK;
    static float scale_gemm(const Op& o) { return o.scaleGemm_; }
    static float scale_relu(const Op& o) { return o.scaleRelu_; }
};

inline void throw_on(int status, const char* what)
{
    if(status != CKX_OK)
        throw std::runtime_error(std::string(what) + ": " + ckx_last_error());
}

} // namespace ckx

namespace ck {
namespace tensor_operation {
namespace device {

struct BaseArgument
{
    virtual ~BaseArgument() {}
    void* p_workspace_ = nullptr; // optional device scratch, GetWorkSpaceSize() bytes (split-K)
};

struct BaseInvoker
{
    virtual float Run(const BaseArgument*, const StreamConfig& = StreamConfig{}) { return 0.f; }
    virtual ~BaseInvoker() {}
};

struct BaseOperator
{
    virtual bool IsSupportedArgument(const BaseArgument*) { return false; }
    virtual std::string GetTypeString() const { return ""; }
    virtual size_t GetWorkSpaceSize(const BaseArgument*) const { return 0; }
    virtual void SetWorkSpacePointer(BaseArgument* p_arg, void* p_workspace) const
    {
        p_arg->p_workspace_ = p_workspace;
    }
    virtual ~BaseOperator() {}
};

// ------------------------------------------------------------------ interfaces
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceGemm : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M, index_t N, index_t K,
                        index_t StrideA, index_t StrideB, index_t StrideC, AElementwiseOperation a_element_op,
                        BElementwiseOperation b_element_op, CElementwiseOperation c_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()                                   = 0;
};

template <typename InElementwiseOperation, typename WeiElementwiseOperation, typename OutElementwiseOperation>
struct DeviceConvFwd : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, index_t N, index_t K, index_t C,
                        std::vector<index_t> input_spatial_lengths, std::vector<index_t> filter_spatial_lengths,
                        std::vector<index_t> output_spatial_lengths, std::vector<index_t> conv_filter_strides,
                        std::vector<index_t> conv_filter_dilations, std::vector<index_t> input_left_pads,
                        std::vector<index_t> input_right_pads, InElementwiseOperation in_element_op,
                        WeiElementwiseOperation wei_element_op, OutElementwiseOperation out_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()                                          = 0;
};

template <typename ALayout, typename B0Layout, typename B1Layout, typename CLayout, typename ADataType,
          typename B0DataType, typename B1DataType, typename CDataType, typename AElementwiseOperation,
          typename B0ElementwiseOperation, typename Acc0ElementwiseOperation, typename B1ElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceBatchedGemmGemm : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, index_t M, index_t N,
                        index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0, index_t StrideB1,
                        index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0, index_t BatchStrideB1,
                        index_t BatchStrideC, AElementwiseOperation a_element_op,
                        B0ElementwiseOperation b0_element_op, Acc0ElementwiseOperation acc0_element_op,
                        B1ElementwiseOperation b1_element_op, CElementwiseOperation c_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()                                     = 0;
};

// upstream device_batched_gemm_softmax_gemm.hpp:15-62
template <typename ALayout, typename B0Layout, typename B1Layout, typename CLayout, typename ADataType,
          typename B0DataType, typename B1DataType, typename CDataType, typename AElementwiseOperation,
          typename B0ElementwiseOperation, typename Acc0ElementwiseOperation, typename B1ElementwiseOperation,
          typename CElementwiseOperation, bool MaskOutUpperTriangle>
struct DeviceBatchedGemmSoftmaxGemm : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, index_t M, index_t N,
                        index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0, index_t StrideB1,
                        index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0, index_t BatchStrideB1,
                        index_t BatchStrideC, AElementwiseOperation a_element_op,
                        B0ElementwiseOperation b0_element_op, Acc0ElementwiseOperation acc0_element_op,
                        B1ElementwiseOperation b1_element_op, CElementwiseOperation c_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()                                     = 0;
};

// device_batched_gemm.hpp:24-45
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceBatchedGemm : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M, index_t N, index_t K,
                        index_t StrideA, index_t StrideB, index_t StrideC, index_t BatchStrideA,
                        index_t BatchStrideB, index_t BatchStrideC, index_t Batch,
                        AElementwiseOperation a_element_op, BElementwiseOperation b_element_op,
                        CElementwiseOperation c_element_op)    = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer() = 0;
};

// device_gemm_splitk.hpp:14-39
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceGemmSplitK : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M, index_t N, index_t K,
                        index_t StrideA, index_t StrideB, index_t StrideC, AElementwiseOperation a_element_op,
                        BElementwiseOperation b_element_op, CElementwiseOperation c_element_op,
                        index_t KBatch)                       = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer() = 0;
};

// device_gemm_multiple_d.hpp:14-55
template <typename ALayout, typename BLayout, typename DELayout, typename ADataType, typename BDataType,
          typename DsDataType, typename EDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CDEElementwiseOperation>
struct DeviceGemmMultipleD : public BaseOperator
{
    static constexpr index_t NumDTensor = DsDataType::Size();
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, std::array<const void*, NumDTensor> p_ds, void* p_e,
                        index_t M, index_t N, index_t K, index_t StrideA, index_t StrideB,
                        std::array<index_t, NumDTensor> StrideDs, index_t StrideE, AElementwiseOperation a_element_op,
                        BElementwiseOperation b_element_op, CDEElementwiseOperation cde_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()                                       = 0;
};

// device_conv_fwd_bias_activation.hpp:18-41
template <typename InElementwiseOperation, typename WeiElementwiseOperation, typename OutElementwiseOperation>
struct DeviceConvFwdBiasActivation : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, const void* p_bias, index_t N, index_t K,
                        index_t C, std::vector<index_t> input_spatial_lengths,
                        std::vector<index_t> filter_spatial_lengths, std::vector<index_t> output_spatial_lengths,
                        std::vector<index_t> conv_filter_strides, std::vector<index_t> conv_filter_dilations,
                        std::vector<index_t> input_left_pads, std::vector<index_t> input_right_pads,
                        InElementwiseOperation in_element_op, WeiElementwiseOperation wei_element_op,
                        OutElementwiseOperation out_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()  = 0;
};

// device_conv_fwd_bias_activation_add.hpp
template <typename InElementwiseOperation, typename WeiElementwiseOperation, typename OutElementwiseOperation>
struct DeviceConvFwdBiasActivationAdd : public BaseOperator
{
    virtual std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, const void* p_bias, const void* p_resi,
                        index_t N, index_t K, index_t C, std::vector<index_t> input_spatial_lengths,
                        std::vector<index_t> filter_spatial_lengths, std::vector<index_t> output_spatial_lengths,
                        std::vector<index_t> conv_filter_strides, std::vector<index_t> conv_filter_dilations,
                        std::vector<index_t> input_left_pads, std::vector<index_t> input_right_pads,
                        InElementwiseOperation in_element_op, WeiElementwiseOperation wei_element_op,
                        OutElementwiseOperation out_element_op) = 0;
    virtual std::unique_ptr<BaseInvoker> MakeInvokerPointer()  = 0;
};

// ------------------------------------------------------------------- common invoker
namespace detail {

// launch_and_time_kernel (include/ck/device_utility/kernel_launch.hpp:13-74): timed mode runs
// the launch nwarmup_ + nrepeat_ times and returns the mean milliseconds; otherwise one
// asynchronous launch and 0.
template <typename Argument, int (*Supported)(const Argument&, int), int (*Launch)(const Argument&, int, void*)>
struct InvokerT : public BaseInvoker
{
    explicit InvokerT(int instance) : instance_(instance) {}
    float Run(const Argument& arg, const StreamConfig& sc = StreamConfig{})
    {
        if(Supported(arg, instance_) != CKX_OK)
            throw std::runtime_error(std::string("wrong! the device operator has invalid setting: ") +
                                     ckx_last_error());
        if(!sc.time_kernel_)
        {
            ckx::throw_on(Launch(arg, instance_, sc.stream_id_), "HIP runtime error");
            return 0.f;
        }
        struct Ctx
        {
            const Argument* a;
            int inst;
            void* s;
        } ctx{&arg, instance_, sc.stream_id_};
        float ms = 0.f;
        ckx::throw_on(ckx_time_launches(
                          [](void* u) {
                              auto* c = static_cast<Ctx*>(u);
                              return Launch(*c->a, c->inst, c->s);
                          },
                          &ctx, sc.nwarmup_, sc.nrepeat_, sc.stream_id_, &ms),
                      "HIP runtime error");
        return ms;
    }
    float Run(const BaseArgument* p_arg, const StreamConfig& sc = StreamConfig{}) override
    {
        const auto* a = dynamic_cast<const Argument*>(p_arg);
        if(!a)
            throw std::runtime_error("wrong! argument does not belong to this device operator");
        return Run(*a, sc);
    }
    int instance_;
};

template <typename T>
struct DTypeOf;
template <>
struct DTypeOf<int8_t>
{
    static constexpr bool is_i8 = true;
};
template <>
struct DTypeOf<half_t>
{
    static constexpr bool is_i8 = false;
};
template <>
struct DTypeOf<bhalf_t>
{
    static constexpr bool is_i8 = false;
};

} // namespace detail

// ------------------------------------------------------------------------ GEMM
// One instance (tile configuration) of the MFMA GEMM. instance = CKX_INSTANCE_AUTO lets the
// library choose by problem shape.
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceGemmMfma : public DeviceGemm<ALayout, BLayout, CLayout, ADataType, BDataType, CDataType,
                                          AElementwiseOperation, BElementwiseOperation, CElementwiseOperation>
{
    static_assert(std::is_same_v<ADataType, BDataType> && std::is_same_v<ADataType, CDataType>,
                  "A, B and C share one data type (int8_t, half_t or bhalf_t)");
    static_assert(std::is_same_v<AElementwiseOperation, element_wise::PassThrough> &&
                      std::is_same_v<BElementwiseOperation, element_wise::PassThrough>,
                  "A/B element-wise operations other than PassThrough are not built");
    static constexpr bool is_i8   = detail::DTypeOf<ADataType>::is_i8;
    static constexpr bool is_bf16 = std::is_same_v<ADataType, bhalf_t>;
    using Epi                   = ckx::EpilogueOf<CElementwiseOperation>;
    static_assert(is_i8 || Epi::kind == CKX_EPI_PASSTHROUGH, "fp16 GEMM only has the PassThrough epilogue");

    struct Argument : public BaseArgument
    {
        const void* p_a;
        const void* p_b;
        void* p_c;
        index_t M, N, K, StrideA, StrideB, StrideC;
        CElementwiseOperation c_element_op;
        Argument(const void* a, const void* b, void* c, index_t m, index_t n, index_t k, index_t sa, index_t sb,
                 index_t sc, CElementwiseOperation cop)
            : p_a(a), p_b(b), p_c(c), M(m), N(n), K(k), StrideA(sa), StrideB(sb), StrideC(sc), c_element_op(cop)
        {
        }
    };

    static int Supported(const Argument& a, int inst)
    {
        if constexpr(is_i8)
            return ckx_gemm_i8_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                                            BLayout::code, CLayout::code, Epi::kind, inst);
        else if constexpr(is_bf16)
            return ckx_gemm_bf16_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                                              BLayout::code, CLayout::code, inst);
        else
            return ckx_gemm_f16_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                                             BLayout::code, CLayout::code, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? WorkSpaceBytes(a, inst) : 0;
        if constexpr(is_i8)
            return ckx_gemm_i8(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                               BLayout::code, CLayout::code, Epi::kind, Epi::scale_gemm(a.c_element_op),
                               Epi::scale_relu(a.c_element_op), inst, a.p_workspace_, ws_bytes, stream);
        else if constexpr(is_bf16)
            return ckx_gemm_bf16(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                                 BLayout::code, CLayout::code, inst, a.p_workspace_, ws_bytes, stream);
        else
            return ckx_gemm_f16(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC, ALayout::code,
                                BLayout::code, CLayout::code, inst, a.p_workspace_, ws_bytes, stream);
    }
    static int64_t WorkSpaceBytes(const Argument& a, int inst)
    {
        return is_i8     ? ckx_gemm_i8_workspace_bytes(a.M, a.N, a.K, inst)
               : is_bf16 ? ckx_gemm_bf16_workspace_bytes(a.M, a.N, a.K, inst)
                         : ckx_gemm_f16_workspace_bytes(a.M, a.N, a.K, inst);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a ? (size_t)WorkSpaceBytes(*a, instance_) : 0;
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceGemmMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}

    static Argument MakeArgument(const ADataType* p_a, const BDataType* p_b, CDataType* p_c, index_t M, index_t N,
                                 index_t K, index_t StrideA, index_t StrideB, index_t StrideC,
                                 AElementwiseOperation, BElementwiseOperation, CElementwiseOperation c_element_op)
    {
        return Argument{p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, c_element_op};
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }

    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument> MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M,
                                                      index_t N, index_t K, index_t StrideA, index_t StrideB,
                                                      index_t StrideC, AElementwiseOperation,
                                                      BElementwiseOperation,
                                                      CElementwiseOperation c_element_op) override
    {
        return std::make_unique<Argument>(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, c_element_op);
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        const int op = is_i8 ? CKX_OP_GEMM_I8 : is_bf16 ? CKX_OP_GEMM_BF16 : CKX_OP_GEMM_F16;
        std::string name = instance_ == CKX_INSTANCE_AUTO ? is_i8     ? "DeviceGemm_i8_i8_i8_mk_nk_mn<auto>"
                                                            : is_bf16 ? "DeviceGemm_bf16_bf16_bf16_mk_nk_mn<auto>"
                                                                      : "DeviceGemm_f16_f16_f16_mk_nk_mn<auto>"
                                                          : ckx_instance_name(op, instance_);
        // the library lists one set of instances for all A / B layouts: put this operator's layouts in the name
        const std::string tag = std::string(std::is_same_v<ALayout, tensor_layout::gemm::RowMajor> ? "mk_" : "km_") +
                                (std::is_same_v<BLayout, tensor_layout::gemm::RowMajor> ? "kn" : "nk");
        const auto pos = name.find("mk_nk");
        if(pos != std::string::npos)
            name.replace(pos, 5, tag);
        return name;
    }
    int instance_;
};

// ------------------------------------------------------------------------ conv2d fwd
template <typename InDataType, typename WeiDataType, typename OutDataType, typename InElementwiseOperation,
          typename WeiElementwiseOperation, typename OutElementwiseOperation>
struct DeviceConv2dFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
    : public DeviceConvFwd<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>
{
    static_assert(std::is_same_v<InDataType, WeiDataType> && std::is_same_v<InDataType, OutDataType>,
                  "input, weight and output share one data type (int8_t or half_t)");
    static constexpr bool is_i8 = detail::DTypeOf<InDataType>::is_i8;
    using Epi                   = ckx::EpilogueOf<OutElementwiseOperation>;
    static constexpr int op_code = is_i8 ? CKX_OP_CONV2D_FWD_I8 : CKX_OP_CONV2D_FWD_F16;

    struct Argument : public BaseArgument
    {
        const void* p_in;
        const void* p_wei;
        void* p_out;
        ckx_conv2d_desc desc;
        bool two_d;
        OutElementwiseOperation out_element_op;
        Argument(const void* in, const void* wei, void* out, index_t N, index_t K, index_t C,
                 const std::vector<index_t>& isp, const std::vector<index_t>& fsp, const std::vector<index_t>& osp,
                 const std::vector<index_t>& st, const std::vector<index_t>& dl, const std::vector<index_t>& lp,
                 const std::vector<index_t>& rp, OutElementwiseOperation oop)
            : p_in(in), p_wei(wei), p_out(out), desc{}, out_element_op(oop)
        {
            two_d = isp.size() == 2 && fsp.size() == 2 && osp.size() == 2 && st.size() == 2 && dl.size() == 2 &&
                    lp.size() == 2 && rp.size() == 2;
            if(two_d)
                desc = ckx_conv2d_desc{N,     K,     C,     isp[0], isp[1], fsp[0], fsp[1], osp[0], osp[1],
                                       st[0], st[1], dl[0], dl[1],  lp[0],  lp[1],  rp[0],  rp[1]};
        }
    };
    static int Supported(const Argument& a, int inst)
    {
        if(!a.two_d)
            return CKX_UNSUPPORTED;
        return ckx_conv2d_fwd_is_supported(op_code, &a.desc, Epi::kind, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? ckx_conv2d_fwd_workspace_bytes(op_code, &a.desc, inst) : 0;
        if constexpr(is_i8)
            return ckx_conv2d_fwd_i8(a.p_in, a.p_wei, a.p_out, &a.desc, Epi::kind,
                                     Epi::scale_gemm(a.out_element_op), Epi::scale_relu(a.out_element_op), inst,
                                     a.p_workspace_, ws_bytes, stream);
        else
            return ckx_conv2d_fwd_f16(a.p_in, a.p_wei, a.p_out, &a.desc, inst, a.p_workspace_, ws_bytes, stream);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && a->two_d ? (size_t)ckx_conv2d_fwd_workspace_bytes(op_code, &a->desc, instance_) : 0;
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceConv2dFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K(int instance = CKX_INSTANCE_AUTO)
        : instance_(instance)
    {
    }
    static Argument MakeArgument(const InDataType* p_in, const WeiDataType* p_wei, OutDataType* p_out, index_t N,
                                 index_t K, index_t C, std::vector<index_t> isp, std::vector<index_t> fsp,
                                 std::vector<index_t> osp, std::vector<index_t> st, std::vector<index_t> dl,
                                 std::vector<index_t> lp, std::vector<index_t> rp, InElementwiseOperation,
                                 WeiElementwiseOperation, OutElementwiseOperation oop)
    {
        return Argument{p_in, p_wei, p_out, N, K, C, isp, fsp, osp, st, dl, lp, rp, oop};
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, index_t N, index_t K, index_t C,
                        std::vector<index_t> isp, std::vector<index_t> fsp, std::vector<index_t> osp,
                        std::vector<index_t> st, std::vector<index_t> dl, std::vector<index_t> lp,
                        std::vector<index_t> rp, InElementwiseOperation, WeiElementwiseOperation,
                        OutElementwiseOperation oop) override
    {
        return std::make_unique<Argument>(p_in, p_wei, p_out, N, K, C, isp, fsp, osp, st, dl, lp, rp, oop);
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        if(instance_ == CKX_INSTANCE_AUTO)
            return is_i8 ? "DeviceConv2dFwd_i8_nhwc_kyxc_nhwk<auto>" : "DeviceConv2dFwd_f16_nhwc_kyxc_nhwk<auto>";
        return ckx_instance_name(op_code, instance_);
    }
    int instance_;
};

// ------------------------------------------------------------------ conv fwd, 1 / 2 / 3 spatial dimensions
// DeviceConvNDFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<..., NumDimSpatial>
// (include/ck/tensor_operation/gpu/device/device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp:76-1046): NWC / NHWC / NDHWC
// input, KXC / KYXC / KZYXC weight, NWK / NHWK / NDHWK output; every vector has NumDimSpatial entries.
template <typename InDataType, typename WeiDataType, typename OutDataType, typename InElementwiseOperation,
          typename WeiElementwiseOperation, typename OutElementwiseOperation, int NumDimSpatial>
struct DeviceConvNDFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
    : public DeviceConvFwd<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>
{
    static_assert(std::is_same_v<InDataType, WeiDataType> && std::is_same_v<InDataType, OutDataType>,
                  "input, weight and output share one data type (int8_t or half_t)");
    static_assert(NumDimSpatial >= 1 && NumDimSpatial <= 3, "1, 2 or 3 spatial dimensions");
    static constexpr bool is_i8 = detail::DTypeOf<InDataType>::is_i8;
    using Epi                   = ckx::EpilogueOf<OutElementwiseOperation>;
    static constexpr int op_code = is_i8 ? CKX_OP_CONV2D_FWD_I8 : CKX_OP_CONV2D_FWD_F16;

    struct Argument : public BaseArgument
    {
        const void* p_in;
        const void* p_wei;
        void* p_out;
        ckx_convnd_desc desc;
        bool dims_ok;
        OutElementwiseOperation out_element_op;
        Argument(const void* in, const void* wei, void* out, index_t N, index_t K, index_t C,
                 const std::vector<index_t>& isp, const std::vector<index_t>& fsp, const std::vector<index_t>& osp,
                 const std::vector<index_t>& st, const std::vector<index_t>& dl, const std::vector<index_t>& lp,
                 const std::vector<index_t>& rp, OutElementwiseOperation oop)
            : p_in(in), p_wei(wei), p_out(out), desc{}, out_element_op(oop)
        {
            constexpr std::size_t nd = NumDimSpatial;
            dims_ok = isp.size() == nd && fsp.size() == nd && osp.size() == nd && st.size() == nd && dl.size() == nd &&
                      lp.size() == nd && rp.size() == nd;
            desc.ndim = NumDimSpatial, desc.N = N, desc.K = K, desc.C = C;
            for(std::size_t i = 0; dims_ok && i < nd; ++i)
            {
                desc.in[i] = isp[i], desc.filter[i] = fsp[i], desc.out[i] = osp[i], desc.stride[i] = st[i];
                desc.dilation[i] = dl[i], desc.pad_left[i] = lp[i], desc.pad_right[i] = rp[i];
            }
        }
    };
    static int Supported(const Argument& a, int inst)
    {
        if(!a.dims_ok)
            return CKX_UNSUPPORTED;
        return ckx_convnd_fwd_is_supported(op_code, &a.desc, Epi::kind, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? ckx_convnd_fwd_workspace_bytes(op_code, &a.desc, inst) : 0;
        return ckx_convnd_fwd(op_code, a.p_in, a.p_wei, a.p_out, &a.desc, Epi::kind, Epi::scale_gemm(a.out_element_op),
                              Epi::scale_relu(a.out_element_op), inst, a.p_workspace_, ws_bytes, stream);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && a->dims_ok ? (size_t)ckx_convnd_fwd_workspace_bytes(op_code, &a->desc, instance_) : 0;
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceConvNDFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K(int instance = CKX_INSTANCE_AUTO)
        : instance_(instance)
    {
    }
    static Argument MakeArgument(const InDataType* p_in, const WeiDataType* p_wei, OutDataType* p_out, index_t N,
                                 index_t K, index_t C, std::vector<index_t> isp, std::vector<index_t> fsp,
                                 std::vector<index_t> osp, std::vector<index_t> st, std::vector<index_t> dl,
                                 std::vector<index_t> lp, std::vector<index_t> rp, InElementwiseOperation,
                                 WeiElementwiseOperation, OutElementwiseOperation oop)
    {
        return Argument{p_in, p_wei, p_out, N, K, C, isp, fsp, osp, st, dl, lp, rp, oop};
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, index_t N, index_t K, index_t C,
                        std::vector<index_t> isp, std::vector<index_t> fsp, std::vector<index_t> osp,
                        std::vector<index_t> st, std::vector<index_t> dl, std::vector<index_t> lp,
                        std::vector<index_t> rp, InElementwiseOperation, WeiElementwiseOperation,
                        OutElementwiseOperation oop) override
    {
        return std::make_unique<Argument>(p_in, p_wei, p_out, N, K, C, isp, fsp, osp, st, dl, lp, rp, oop);
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        const std::string nd = "DeviceConv" + std::to_string(NumDimSpatial) + "dFwd";
        if(instance_ == CKX_INSTANCE_AUTO)
            return nd + (is_i8 ? "_i8_channels_last<auto>" : "_f16_channels_last<auto>");
        const char* n = ckx_instance_name(op_code, instance_);
        return nd + ":" + (n ? n : "?");
    }
    int instance_;
};

// ------------------------------------------------------------------ strided batched GEMM
// One launch for all batches: the persistent workgroups walk the C tiles of every batch.
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceBatchedGemmMfma : public DeviceBatchedGemm<ALayout, BLayout, CLayout, ADataType, BDataType, CDataType,
                                                        AElementwiseOperation, BElementwiseOperation,
                                                        CElementwiseOperation>
{
    using Plain = DeviceGemmMfma<ALayout, BLayout, CLayout, ADataType, BDataType, CDataType, AElementwiseOperation,
                                 BElementwiseOperation, CElementwiseOperation>;
    static constexpr bool is_i8 = Plain::is_i8;
    using Epi                   = typename Plain::Epi;
    struct Argument : public Plain::Argument
    {
        index_t BatchStrideA, BatchStrideB, BatchStrideC, Batch;
        Argument(const void* a, const void* b, void* c, index_t m, index_t n, index_t k, index_t sa, index_t sb,
                 index_t sc, index_t bsa, index_t bsb, index_t bsc, index_t batch, CElementwiseOperation cop)
            : Plain::Argument(a, b, c, m, n, k, sa, sb, sc, cop), BatchStrideA(bsa), BatchStrideB(bsb),
              BatchStrideC(bsc), Batch(batch)
        {
        }
    };
    static int Supported(const Argument& a, int inst)
    {
        return ckx_batched_gemm_is_supported(is_i8 ? CKX_OP_GEMM_I8 : CKX_OP_GEMM_F16, a.M, a.N, a.K, a.StrideA,
                                             a.StrideB, a.StrideC, a.BatchStrideA, a.BatchStrideB, a.BatchStrideC,
                                             a.Batch, ALayout::code, BLayout::code, CLayout::code, Epi::kind, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        if constexpr(is_i8)
            return ckx_batched_gemm_i8(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                       a.BatchStrideA, a.BatchStrideB, a.BatchStrideC, a.Batch, ALayout::code,
                                       BLayout::code, CLayout::code, Epi::kind, Epi::scale_gemm(a.c_element_op),
                                       Epi::scale_relu(a.c_element_op), inst, stream);
        else
            return ckx_batched_gemm_f16(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                        a.BatchStrideA, a.BatchStrideB, a.BatchStrideC, a.Batch, ALayout::code,
                                        BLayout::code, CLayout::code, inst, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceBatchedGemmMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const ADataType* p_a, const BDataType* p_b, CDataType* p_c, index_t M, index_t N,
                                 index_t K, index_t StrideA, index_t StrideB, index_t StrideC, index_t BatchStrideA,
                                 index_t BatchStrideB, index_t BatchStrideC, index_t Batch, AElementwiseOperation,
                                 BElementwiseOperation, CElementwiseOperation c_element_op)
    {
        return Argument{p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, BatchStrideA, BatchStrideB, BatchStrideC,
                        Batch, c_element_op};
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M, index_t N, index_t K,
                        index_t StrideA, index_t StrideB, index_t StrideC, index_t BatchStrideA,
                        index_t BatchStrideB, index_t BatchStrideC, index_t Batch, AElementwiseOperation,
                        BElementwiseOperation, CElementwiseOperation c_element_op) override
    {
        return std::make_unique<Argument>(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, BatchStrideA,
                                          BatchStrideB, BatchStrideC, Batch, c_element_op);
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override { return Plain(instance_).GetTypeString() + " + Batched"; }
    int instance_;
};

// ------------------------------------------------------------------ split-K GEMM
// KBatch runs over K, raw accumulators in the workspace (GetWorkSpaceSize / SetWorkSpacePointer,
// REQUIRED for KBatch > 1), summed in run order by a second kernel: deterministic, int8 bit-identical
// to the unsplit operator.
template <typename ALayout, typename BLayout, typename CLayout, typename ADataType, typename BDataType,
          typename CDataType, typename AElementwiseOperation, typename BElementwiseOperation,
          typename CElementwiseOperation>
struct DeviceGemmSplitKMfma : public DeviceGemmSplitK<ALayout, BLayout, CLayout, ADataType, BDataType, CDataType,
                                                      AElementwiseOperation, BElementwiseOperation,
                                                      CElementwiseOperation>
{
    using Plain = DeviceGemmMfma<ALayout, BLayout, CLayout, ADataType, BDataType, CDataType, AElementwiseOperation,
                                 BElementwiseOperation, CElementwiseOperation>;
    static constexpr bool is_i8 = Plain::is_i8;
    using Epi                   = typename Plain::Epi;
    struct Argument : public Plain::Argument
    {
        index_t KBatch;
        Argument(const void* a, const void* b, void* c, index_t m, index_t n, index_t k, index_t sa, index_t sb,
                 index_t sc, CElementwiseOperation cop, index_t kbatch)
            : Plain::Argument(a, b, c, m, n, k, sa, sb, sc, cop), KBatch(kbatch)
        {
        }
    };
    static int64_t WorkSpaceBytes(const Argument& a)
    {
        return ckx_gemm_splitk_workspace_bytes(is_i8 ? CKX_OP_GEMM_I8 : CKX_OP_GEMM_F16, a.M, a.N, a.K, a.KBatch);
    }
    static int Supported(const Argument& a, int inst)
    {
        if(a.KBatch < 1 || a.KBatch > 8 || inst >= ckx_num_instances(CKX_OP_GEMM_SPLITK))
            return CKX_UNSUPPORTED;
        return Plain::Supported(a, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? WorkSpaceBytes(a) : 0;
        if constexpr(is_i8)
            return ckx_gemm_i8_splitk(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                      ALayout::code, BLayout::code, CLayout::code, Epi::kind,
                                      Epi::scale_gemm(a.c_element_op), Epi::scale_relu(a.c_element_op), inst,
                                      a.KBatch, a.p_workspace_, ws_bytes, stream);
        else
            return ckx_gemm_f16_splitk(a.p_a, a.p_b, a.p_c, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideC,
                                       ALayout::code, BLayout::code, CLayout::code, inst, a.KBatch, a.p_workspace_,
                                       ws_bytes, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceGemmSplitKMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const ADataType* p_a, const BDataType* p_b, CDataType* p_c, index_t M, index_t N,
                                 index_t K, index_t StrideA, index_t StrideB, index_t StrideC,
                                 AElementwiseOperation, BElementwiseOperation, CElementwiseOperation c_element_op,
                                 index_t KBatch)
    {
        return Argument{p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, c_element_op, KBatch};
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a ? (size_t)WorkSpaceBytes(*a) : 0;
    }
    std::unique_ptr<BaseArgument> MakeArgumentPointer(const void* p_a, const void* p_b, void* p_c, index_t M,
                                                      index_t N, index_t K, index_t StrideA, index_t StrideB,
                                                      index_t StrideC, AElementwiseOperation,
                                                      BElementwiseOperation, CElementwiseOperation c_element_op,
                                                      index_t KBatch) override
    {
        return std::make_unique<Argument>(p_a, p_b, p_c, M, N, K, StrideA, StrideB, StrideC, c_element_op, KBatch);
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override { return Plain(instance_).GetTypeString() + " + SplitK"; }
    int instance_;
};

// ------------------------------------------------ GEMM with fused D operands (fp16)
// CDE operation: AddRelu (one D: E = relu(half(C) + D0), example 03), AddReluAdd (two Ds: E = relu(C + D0) + D1 in
// fp32), Bilinear (one D: E = alpha * C + beta * D0, example 02) or AddAddFastGelu (two Ds: E = fast_gelu(C + D0 + D1),
// example 04). A D stride of 0 broadcasts one row (a bias vector).
template <typename ALayout, typename BLayout, typename DELayout, typename DsDataType,
          typename CDEElementwiseOperation>
struct DeviceGemmMultipleDMfma
    : public DeviceGemmMultipleD<ALayout, BLayout, DELayout, half_t, half_t, DsDataType, half_t,
                                 element_wise::PassThrough, element_wise::PassThrough, CDEElementwiseOperation>
{
    static constexpr index_t NumDTensor = DsDataType::Size();
    static constexpr bool is_add_relu   = std::is_same_v<CDEElementwiseOperation, element_wise::AddRelu>;
    static constexpr bool is_bilinear   = std::is_same_v<CDEElementwiseOperation, element_wise::Bilinear>;
    static constexpr bool is_gelu       = std::is_same_v<CDEElementwiseOperation, element_wise::AddAddFastGelu>;
    static_assert(((is_add_relu || is_bilinear) && NumDTensor == 1) ||
                      ((std::is_same_v<CDEElementwiseOperation, element_wise::AddReluAdd> || is_gelu) && NumDTensor == 2),
                  "built CDE operations: AddRelu and Bilinear with one D tensor, AddReluAdd and AddAddFastGelu with two");
    static constexpr int cde_code = is_add_relu   ? CKX_EPI_CSHUFFLE_ADD_RELU
                                    : is_bilinear ? CKX_EPI_BILINEAR
                                    : is_gelu     ? CKX_EPI_ADD_ADD_FASTGELU
                                                  : CKX_EPI_ADD_RELU_ADD;
    using Pass                    = element_wise::PassThrough;

    struct Argument : public BaseArgument
    {
        const void *p_a, *p_b, *p_d0, *p_d1;
        void* p_e;
        index_t M, N, K, StrideA, StrideB, StrideD0, StrideD1, StrideE;
        CDEElementwiseOperation cde_element_op_;
    };
    static int Supported(const Argument& a, int inst)
    {
        return ckx_gemm_f16_multiple_d_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideD0, a.StrideD1,
                                                    a.StrideE, ALayout::code, BLayout::code, DELayout::code,
                                                    cde_code, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? ckx_gemm_f16_workspace_bytes(a.M, a.N, a.K, inst) : 0;
        if constexpr(is_bilinear)
            return ckx_gemm_f16_bilinear(a.p_a, a.p_b, a.p_d0, a.p_e, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideD0,
                                         a.StrideE, ALayout::code, BLayout::code, DELayout::code,
                                         a.cde_element_op_.alpha_, a.cde_element_op_.beta_, inst, a.p_workspace_,
                                         ws_bytes, stream);
        else
            return ckx_gemm_f16_multiple_d(a.p_a, a.p_b, a.p_d0, a.p_d1, a.p_e, a.M, a.N, a.K, a.StrideA, a.StrideB,
                                           a.StrideD0, a.StrideD1, a.StrideE, ALayout::code, BLayout::code,
                                           DELayout::code, cde_code, inst, a.p_workspace_, ws_bytes, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceGemmMultipleDMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const void* p_a, const void* p_b, std::array<const void*, NumDTensor> p_ds,
                                 void* p_e, index_t M, index_t N, index_t K, index_t StrideA, index_t StrideB,
                                 std::array<index_t, NumDTensor> StrideDs, index_t StrideE, Pass = {}, Pass = {},
                                 CDEElementwiseOperation cde_element_op = {})
    {
        Argument a;
        a.cde_element_op_ = cde_element_op;
        a.p_a = p_a, a.p_b = p_b, a.p_e = p_e;
        a.p_d0 = p_ds[0], a.StrideD0 = StrideDs[0];
        a.p_d1 = NumDTensor > 1 ? p_ds[NumDTensor - 1] : nullptr, a.StrideD1 = NumDTensor > 1 ? StrideDs[NumDTensor - 1] : 0;
        a.M = M, a.N = N, a.K = K, a.StrideA = StrideA, a.StrideB = StrideB, a.StrideE = StrideE;
        return a;
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a ? (size_t)ckx_gemm_f16_workspace_bytes(a->M, a->N, a->K, instance_) : 0;
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, std::array<const void*, NumDTensor> p_ds, void* p_e,
                        index_t M, index_t N, index_t K, index_t StrideA, index_t StrideB,
                        std::array<index_t, NumDTensor> StrideDs, index_t StrideE, Pass, Pass,
                        CDEElementwiseOperation cde_element_op) override
    {
        return std::make_unique<Argument>(MakeArgument(p_a, p_b, p_ds, p_e, M, N, K, StrideA, StrideB, StrideDs, StrideE,
                                                       Pass{}, Pass{}, cde_element_op));
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        const std::string base = instance_ == CKX_INSTANCE_AUTO ? std::string("DeviceGemm_f16_f16_f16_mk_nk_mn<auto>")
                                                                : std::string(ckx_instance_name(CKX_OP_GEMM_F16, instance_));
        return base + (is_add_relu ? " + AddRelu" : is_bilinear ? " + Bilinear" : is_gelu ? " + AddAddFastGelu" : " + AddReluAdd");
    }
    int instance_;
};

// ------------------------------------------------ int8 GEMM with one requant scale per output column
// DeviceGemmMultipleD<..., int8_t, int8_t, Tuple<float>, int8_t, PassThrough, PassThrough,
// Activation_Mul2_Clamp<Activation>> (device_gemm_multiple_d.hpp:14-55): D0 is a row of N floats, stride 0.
template <typename ALayout, typename BLayout, typename DELayout, typename Activation>
struct DeviceGemmMultipleDInt8Mfma
    : public DeviceGemmMultipleD<ALayout, BLayout, DELayout, int8_t, int8_t, Tuple<float>, int8_t,
                                 element_wise::PassThrough, element_wise::PassThrough,
                                 element_wise::Activation_Mul2_Clamp<Activation>>
{
    static constexpr bool is_relu = std::is_same_v<Activation, element_wise::Relu>;
    static_assert(is_relu || std::is_same_v<Activation, element_wise::PassThrough>, "built activations: PassThrough, Relu");
    static constexpr int cde_code = is_relu ? CKX_EPI_RELU_MUL2_CLAMP : CKX_EPI_MUL2_CLAMP;
    using Pass                    = element_wise::PassThrough;
    using CDEOp                   = element_wise::Activation_Mul2_Clamp<Activation>;

    struct Argument : public BaseArgument
    {
        const void *p_a, *p_b, *p_d0;
        void* p_e;
        index_t M, N, K, StrideA, StrideB, StrideD0, StrideE;
    };
    static int Supported(const Argument& a, int inst)
    {
        return ckx_gemm_i8_multiple_d_is_supported(a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideD0, a.StrideE,
                                                   ALayout::code, BLayout::code, DELayout::code, cde_code, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        const int64_t ws_bytes = a.p_workspace_ ? ckx_gemm_i8_workspace_bytes(a.M, a.N, a.K, inst) : 0;
        return ckx_gemm_i8_multiple_d(a.p_a, a.p_b, a.p_d0, a.p_e, a.M, a.N, a.K, a.StrideA, a.StrideB, a.StrideD0,
                                      a.StrideE, ALayout::code, BLayout::code, DELayout::code, cde_code, inst,
                                      a.p_workspace_, ws_bytes, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceGemmMultipleDInt8Mfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const void* p_a, const void* p_b, std::array<const void*, 1> p_ds, void* p_e,
                                 index_t M, index_t N, index_t K, index_t StrideA, index_t StrideB,
                                 std::array<index_t, 1> StrideDs, index_t StrideE, Pass = {}, Pass = {}, CDEOp = {})
    {
        Argument a;
        a.p_a = p_a, a.p_b = p_b, a.p_d0 = p_ds[0], a.p_e = p_e;
        a.M = M, a.N = N, a.K = K, a.StrideA = StrideA, a.StrideB = StrideB, a.StrideD0 = StrideDs[0], a.StrideE = StrideE;
        return a;
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a ? (size_t)ckx_gemm_i8_workspace_bytes(a->M, a->N, a->K, instance_) : 0;
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b, std::array<const void*, 1> p_ds, void* p_e, index_t M,
                        index_t N, index_t K, index_t StrideA, index_t StrideB, std::array<index_t, 1> StrideDs,
                        index_t StrideE, Pass, Pass, CDEOp) override
    {
        return std::make_unique<Argument>(MakeArgument(p_a, p_b, p_ds, p_e, M, N, K, StrideA, StrideB, StrideDs, StrideE));
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        const std::string base = instance_ == CKX_INSTANCE_AUTO ? std::string("DeviceGemm_i8_i8_i8_mk_nk_mn<auto>")
                                                                : std::string(ckx_instance_name(CKX_OP_GEMM_I8, instance_));
        return base + (is_relu ? " + Relu_Mul2_Clamp" : " + Mul2_Clamp");
    }
    int instance_;
};

// ------------------------------------------ conv2d fwd + bias + ReLU (+ residual), fp16
namespace detail {
struct ConvBiasArgument : public BaseArgument
{
    const void *p_in, *p_wei, *p_bias, *p_resi;
    void* p_out;
    ckx_conv2d_desc desc;
    bool two_d;
    int out_op;
    ConvBiasArgument(const void* in, const void* wei, void* out, const void* bias, const void* resi, int op,
                     index_t N, index_t K, index_t C, const std::vector<index_t>& isp,
                     const std::vector<index_t>& fsp, const std::vector<index_t>& osp, const std::vector<index_t>& st,
                     const std::vector<index_t>& dl, const std::vector<index_t>& lp, const std::vector<index_t>& rp)
        : p_in(in), p_wei(wei), p_bias(bias), p_resi(resi), p_out(out), desc{}, out_op(op)
    {
        two_d = isp.size() == 2 && fsp.size() == 2 && osp.size() == 2 && st.size() == 2 && dl.size() == 2 &&
                lp.size() == 2 && rp.size() == 2;
        if(two_d)
            desc = ckx_conv2d_desc{N,     K,     C,     isp[0], isp[1], fsp[0], fsp[1], osp[0], osp[1],
                                   st[0], st[1], dl[0], dl[1],  lp[0],  lp[1],  rp[0],  rp[1]};
    }
};
inline int conv_bias_supported(const ConvBiasArgument& a, int inst)
{
    return a.two_d ? ckx_conv2d_fwd_is_supported(CKX_OP_CONV2D_FWD_F16, &a.desc, a.out_op, inst) : CKX_UNSUPPORTED;
}
inline int conv_bias_launch(const ConvBiasArgument& a, int inst, void* stream)
{
    const int64_t ws_bytes = a.p_workspace_ ? ckx_conv2d_fwd_workspace_bytes(CKX_OP_CONV2D_FWD_F16, &a.desc, inst) : 0;
    return ckx_conv2d_fwd_bias_activation_f16(a.p_in, a.p_wei, a.p_out, a.p_bias, a.p_resi, &a.desc, a.out_op, inst,
                                              a.p_workspace_, ws_bytes, stream);
}
using ConvBiasInvoker = InvokerT<ConvBiasArgument, &conv_bias_supported, &conv_bias_launch>;

// what the two operators share; Derived supplies the interface base class
template <typename Base>
struct ConvBiasCommon : public Base
{
    using Argument = ConvBiasArgument;
    using Invoker  = ConvBiasInvoker;
    explicit ConvBiasCommon(int instance) : instance_(instance) {}
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return conv_bias_supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    size_t GetWorkSpaceSize(const BaseArgument* p) const override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && a->two_d ? (size_t)ckx_conv2d_fwd_workspace_bytes(CKX_OP_CONV2D_FWD_F16, &a->desc, instance_) : 0;
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    int instance_;
};
} // namespace detail

// DeviceConv2dFwdXdl_C_Shuffle_Bias_Activation_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K (example 06)
template <typename InElementwiseOperation = element_wise::PassThrough,
          typename WeiElementwiseOperation = element_wise::PassThrough,
          typename OutElementwiseOperation = element_wise::AddRelu>
struct DeviceConv2dFwdBiasActivationMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
    : public detail::ConvBiasCommon<
          DeviceConvFwdBiasActivation<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>>
{
    static_assert(std::is_same_v<OutElementwiseOperation, element_wise::AddRelu>, "built output operation: AddRelu");
    using Common = detail::ConvBiasCommon<
        DeviceConvFwdBiasActivation<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>>;
    using Argument = detail::ConvBiasArgument;
    explicit DeviceConv2dFwdBiasActivationMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K(
        int instance = CKX_INSTANCE_AUTO)
        : Common(instance)
    {
    }
    static Argument MakeArgument(const half_t* p_in, const half_t* p_wei, half_t* p_out, const half_t* p_bias,
                                 index_t N, index_t K, index_t C, std::vector<index_t> isp, std::vector<index_t> fsp,
                                 std::vector<index_t> osp, std::vector<index_t> st, std::vector<index_t> dl,
                                 std::vector<index_t> lp, std::vector<index_t> rp, InElementwiseOperation = {},
                                 WeiElementwiseOperation = {}, OutElementwiseOperation = {})
    {
        return Argument{p_in, p_wei, p_out, p_bias, nullptr, CKX_EPI_ADD_RELU, N, K, C, isp, fsp, osp, st, dl, lp, rp};
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, const void* p_bias, index_t N, index_t K,
                        index_t C, std::vector<index_t> isp, std::vector<index_t> fsp, std::vector<index_t> osp,
                        std::vector<index_t> st, std::vector<index_t> dl, std::vector<index_t> lp,
                        std::vector<index_t> rp, InElementwiseOperation, WeiElementwiseOperation,
                        OutElementwiseOperation) override
    {
        return std::make_unique<Argument>(p_in, p_wei, p_out, p_bias, nullptr, CKX_EPI_ADD_RELU, N, K, C, isp, fsp, osp,
                                          st, dl, lp, rp);
    }
    std::string GetTypeString() const override
    {
        return (this->instance_ == CKX_INSTANCE_AUTO ? std::string("DeviceConv2dFwd_f16_nhwc_kyxc_nhwk<auto>")
                                                     : std::string(ckx_instance_name(CKX_OP_CONV2D_FWD_F16, this->instance_))) +
               " + Bias + AddRelu";
    }
};

// ..._Bias_Activation_Add_... (example 07)
template <typename InElementwiseOperation = element_wise::PassThrough,
          typename WeiElementwiseOperation = element_wise::PassThrough,
          typename OutElementwiseOperation = element_wise::AddReluAdd>
struct DeviceConv2dFwdBiasActivationAddMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
    : public detail::ConvBiasCommon<
          DeviceConvFwdBiasActivationAdd<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>>
{
    static_assert(std::is_same_v<OutElementwiseOperation, element_wise::AddReluAdd>,
                  "built output operation: AddReluAdd");
    using Common = detail::ConvBiasCommon<
        DeviceConvFwdBiasActivationAdd<InElementwiseOperation, WeiElementwiseOperation, OutElementwiseOperation>>;
    using Argument = detail::ConvBiasArgument;
    explicit DeviceConv2dFwdBiasActivationAddMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K(
        int instance = CKX_INSTANCE_AUTO)
        : Common(instance)
    {
    }
    static Argument MakeArgument(const half_t* p_in, const half_t* p_wei, half_t* p_out, const half_t* p_bias,
                                 const half_t* p_resi, index_t N, index_t K, index_t C, std::vector<index_t> isp,
                                 std::vector<index_t> fsp, std::vector<index_t> osp, std::vector<index_t> st,
                                 std::vector<index_t> dl, std::vector<index_t> lp, std::vector<index_t> rp,
                                 InElementwiseOperation = {}, WeiElementwiseOperation = {},
                                 OutElementwiseOperation = {})
    {
        return Argument{p_in, p_wei, p_out, p_bias, p_resi, CKX_EPI_ADD_RELU_ADD, N, K, C, isp, fsp, osp, st, dl, lp, rp};
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_in, const void* p_wei, void* p_out, const void* p_bias, const void* p_resi,
                        index_t N, index_t K, index_t C, std::vector<index_t> isp, std::vector<index_t> fsp,
                        std::vector<index_t> osp, std::vector<index_t> st, std::vector<index_t> dl,
                        std::vector<index_t> lp, std::vector<index_t> rp, InElementwiseOperation,
                        WeiElementwiseOperation, OutElementwiseOperation) override
    {
        return std::make_unique<Argument>(p_in, p_wei, p_out, p_bias, p_resi, CKX_EPI_ADD_RELU_ADD, N, K, C, isp, fsp,
                                          osp, st, dl, lp, rp);
    }
    std::string GetTypeString() const override
    {
        return (this->instance_ == CKX_INSTANCE_AUTO ? std::string("DeviceConv2dFwd_f16_nhwc_kyxc_nhwk<auto>")
                                                     : std::string(ckx_instance_name(CKX_OP_CONV2D_FWD_F16, this->instance_))) +
               " + Bias + AddReluAdd";
    }
};

// -------------------------------------------------------------------- GEMM-GEMM
template <typename AElementwiseOperation = element_wise::PassThrough,
          typename B0ElementwiseOperation = element_wise::PassThrough,
          typename Acc0ElementwiseOperation = element_wise::PassThrough,
          typename B1ElementwiseOperation = element_wise::PassThrough,
          typename CElementwiseOperation = element_wise::PassThrough>
struct DeviceBatchedGemmGemmMfma
    : public DeviceBatchedGemmGemm<tensor_layout::gemm::RowMajor, tensor_layout::gemm::ColumnMajor,
                                   tensor_layout::gemm::RowMajor, tensor_layout::gemm::RowMajor, half_t, half_t,
                                   half_t, half_t, AElementwiseOperation, B0ElementwiseOperation,
                                   Acc0ElementwiseOperation, B1ElementwiseOperation, CElementwiseOperation>
{
    static_assert(std::is_same_v<AElementwiseOperation, element_wise::PassThrough> &&
                      std::is_same_v<B0ElementwiseOperation, element_wise::PassThrough> &&
                      std::is_same_v<Acc0ElementwiseOperation, element_wise::PassThrough> &&
                      std::is_same_v<B1ElementwiseOperation, element_wise::PassThrough> &&
                      std::is_same_v<CElementwiseOperation, element_wise::PassThrough>,
                  "only PassThrough element-wise operations are built");
    struct Argument : public BaseArgument
    {
        const void *p_a, *p_b0, *p_b1;
        void* p_c;
        index_t M, N, K, O, Batch, StrideA, StrideB0, StrideB1, StrideC;
        int64_t BatchStrideA, BatchStrideB0, BatchStrideB1, BatchStrideC;
    };
    static int Supported(const Argument& a, int inst)
    {
        return ckx_batched_gemm_gemm_f16_is_supported(a.M, a.N, a.K, a.O, a.Batch, a.StrideA, a.StrideB0, a.StrideB1,
                                                      a.StrideC, a.BatchStrideA, a.BatchStrideB0, a.BatchStrideB1,
                                                      a.BatchStrideC, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        return ckx_batched_gemm_gemm_f16(a.p_a, a.p_b0, a.p_b1, a.p_c, a.M, a.N, a.K, a.O, a.Batch, a.StrideA,
                                         a.StrideB0, a.StrideB1, a.StrideC, a.BatchStrideA, a.BatchStrideB0,
                                         a.BatchStrideB1, a.BatchStrideC, inst, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceBatchedGemmGemmMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const half_t* p_a, const half_t* p_b0, const half_t* p_b1, half_t* p_c, index_t M,
                                 index_t N, index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0,
                                 index_t StrideB1, index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0,
                                 index_t BatchStrideB1, index_t BatchStrideC, AElementwiseOperation = {},
                                 B0ElementwiseOperation = {}, Acc0ElementwiseOperation = {},
                                 B1ElementwiseOperation = {}, CElementwiseOperation = {})
    {
        Argument a;
        a.p_a = p_a, a.p_b0 = p_b0, a.p_b1 = p_b1, a.p_c = p_c;
        a.M = M, a.N = N, a.K = K, a.O = O, a.Batch = Batch;
        a.StrideA = StrideA, a.StrideB0 = StrideB0, a.StrideB1 = StrideB1, a.StrideC = StrideC;
        a.BatchStrideA = BatchStrideA, a.BatchStrideB0 = BatchStrideB0, a.BatchStrideB1 = BatchStrideB1,
        a.BatchStrideC = BatchStrideC;
        return a;
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, index_t M, index_t N,
                        index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0, index_t StrideB1,
                        index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0, index_t BatchStrideB1,
                        index_t BatchStrideC, AElementwiseOperation, B0ElementwiseOperation,
                        Acc0ElementwiseOperation, B1ElementwiseOperation, CElementwiseOperation) override
    {
        return std::make_unique<Argument>(MakeArgument(
            static_cast<const half_t*>(p_a), static_cast<const half_t*>(p_b0), static_cast<const half_t*>(p_b1),
            static_cast<half_t*>(p_c), M, N, K, O, Batch, StrideA, StrideB0, StrideB1, StrideC, BatchStrideA,
            BatchStrideB0, BatchStrideB1, BatchStrideC));
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        if(instance_ == CKX_INSTANCE_AUTO)
            return "DeviceBatchedGemmGemm_f16_gmk_gnk_gno_gmo<auto>";
        return ckx_instance_name(CKX_OP_BATCHED_GEMM_GEMM, instance_);
    }
    int instance_;
};

// ------------------------------------------------------------- GEMM + softmax + GEMM
// Acc0ElementwiseOperation: element_wise::Scale (or PassThrough = scale 1); MaskOutUpperTriangle as in upstream
template <typename Acc0ElementwiseOperation = element_wise::Scale, bool MaskOutUpperTriangle = false>
struct DeviceBatchedGemmSoftmaxGemmMfma
    : public DeviceBatchedGemmSoftmaxGemm<tensor_layout::gemm::RowMajor, tensor_layout::gemm::ColumnMajor,
                                          tensor_layout::gemm::RowMajor, tensor_layout::gemm::RowMajor, half_t, half_t,
                                          half_t, half_t, element_wise::PassThrough, element_wise::PassThrough,
                                          Acc0ElementwiseOperation, element_wise::PassThrough,
                                          element_wise::PassThrough, MaskOutUpperTriangle>
{
    using Pass = element_wise::PassThrough;
    static_assert(std::is_same_v<Acc0ElementwiseOperation, element_wise::Scale> ||
                      std::is_same_v<Acc0ElementwiseOperation, Pass>,
                  "the score operation is Scale or PassThrough");
    struct Argument : public BaseArgument
    {
        const void *p_a, *p_b0, *p_b1;
        void* p_c;
        index_t M, N, K, O, Batch, StrideA, StrideB0, StrideB1, StrideC;
        int64_t BatchStrideA, BatchStrideB0, BatchStrideB1, BatchStrideC;
        float scale;
    };
    static float ScaleOf(const element_wise::Scale& op) { return op.scale_; }
    static float ScaleOf(const Pass&) { return 1.0f; }
    static int Supported(const Argument& a, int inst)
    {
        return ckx_batched_gemm_softmax_gemm_f16_is_supported(a.M, a.N, a.K, a.O, a.Batch, a.StrideA, a.StrideB0,
                                                              a.StrideB1, a.StrideC, a.BatchStrideA, a.BatchStrideB0,
                                                              a.BatchStrideB1, a.BatchStrideC, a.scale,
                                                              MaskOutUpperTriangle ? 1 : 0, inst);
    }
    static int Launch(const Argument& a, int inst, void* stream)
    {
        return ckx_batched_gemm_softmax_gemm_f16(a.p_a, a.p_b0, a.p_b1, a.p_c, a.M, a.N, a.K, a.O, a.Batch, a.StrideA,
                                                 a.StrideB0, a.StrideB1, a.StrideC, a.BatchStrideA, a.BatchStrideB0,
                                                 a.BatchStrideB1, a.BatchStrideC, a.scale,
                                                 MaskOutUpperTriangle ? 1 : 0, inst, stream);
    }
    using Invoker = detail::InvokerT<Argument, &Supported, &Launch>;

    explicit DeviceBatchedGemmSoftmaxGemmMfma(int instance = CKX_INSTANCE_AUTO) : instance_(instance) {}
    static Argument MakeArgument(const half_t* p_a, const half_t* p_b0, const half_t* p_b1, half_t* p_c, index_t M,
                                 index_t N, index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0,
                                 index_t StrideB1, index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0,
                                 index_t BatchStrideB1, index_t BatchStrideC, Pass = {}, Pass = {},
                                 Acc0ElementwiseOperation acc0_element_op = {}, Pass = {}, Pass = {})
    {
        Argument a;
        a.p_a = p_a, a.p_b0 = p_b0, a.p_b1 = p_b1, a.p_c = p_c;
        a.M = M, a.N = N, a.K = K, a.O = O, a.Batch = Batch;
        a.StrideA = StrideA, a.StrideB0 = StrideB0, a.StrideB1 = StrideB1, a.StrideC = StrideC;
        a.BatchStrideA = BatchStrideA, a.BatchStrideB0 = BatchStrideB0, a.BatchStrideB1 = BatchStrideB1,
        a.BatchStrideC = BatchStrideC;
        a.scale        = ScaleOf(acc0_element_op);
        return a;
    }
    Invoker MakeInvoker() const { return Invoker{instance_}; }
    bool IsSupportedArgument(const Argument& a) const { return Supported(a, instance_) == CKX_OK; }
    bool IsSupportedArgument(const BaseArgument* p) override
    {
        const auto* a = dynamic_cast<const Argument*>(p);
        return a && IsSupportedArgument(*a);
    }
    std::unique_ptr<BaseArgument>
    MakeArgumentPointer(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, index_t M, index_t N,
                        index_t K, index_t O, index_t Batch, index_t StrideA, index_t StrideB0, index_t StrideB1,
                        index_t StrideC, index_t BatchStrideA, index_t BatchStrideB0, index_t BatchStrideB1,
                        index_t BatchStrideC, Pass, Pass, Acc0ElementwiseOperation acc0_element_op, Pass, Pass) override
    {
        return std::make_unique<Argument>(MakeArgument(
            static_cast<const half_t*>(p_a), static_cast<const half_t*>(p_b0), static_cast<const half_t*>(p_b1),
            static_cast<half_t*>(p_c), M, N, K, O, Batch, StrideA, StrideB0, StrideB1, StrideC, BatchStrideA,
            BatchStrideB0, BatchStrideB1, BatchStrideC, Pass{}, Pass{}, acc0_element_op));
    }
    std::unique_ptr<BaseInvoker> MakeInvokerPointer() override { return std::make_unique<Invoker>(instance_); }
    std::string GetTypeString() const override
    {
        if(instance_ == CKX_INSTANCE_AUTO)
            return "DeviceBatchedGemmSoftmaxGemm_f16_gmk_gnk_gno_gmo<auto>";
        return ckx_instance_name(CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM, instance_);
    }
    int instance_;
};

// ------------------------------------------------------------------ instance factory
namespace instance {

template <typename DeviceOp>
struct DeviceOperationInstanceFactory;

template <typename AL, typename BL, typename CL, typename T, typename AOp, typename BOp, typename COp>
struct DeviceOperationInstanceFactory<DeviceGemm<AL, BL, CL, T, T, T, AOp, BOp, COp>>
{
    using DeviceOp = DeviceGemm<AL, BL, CL, T, T, T, AOp, BOp, COp>;
    static std::vector<std::unique_ptr<DeviceOp>> GetInstances()
    {
        std::vector<std::unique_ptr<DeviceOp>> v;
        const int n = ckx_num_instances(CKX_OP_GEMM_F16); // the same list for every data type
        for(int i = 0; i < n; ++i)
            v.push_back(std::make_unique<DeviceGemmMfma<AL, BL, CL, T, T, T, AOp, BOp, COp>>(i));
        return v;
    }
};

// conv: the interface type carries no data type, so the caller names it
// (ConvolutionFwdInstances<T,T,T>::Get<2>(), library/include/ck/library/utility/conv_util.hpp:288-397)
template <typename T, typename InOp, typename WeiOp, typename OutOp>
std::vector<std::unique_ptr<DeviceConvFwd<InOp, WeiOp, OutOp>>> GetConv2dFwdInstances()
{
    std::vector<std::unique_ptr<DeviceConvFwd<InOp, WeiOp, OutOp>>> v;
    const int n = ckx_num_instances(detail::DTypeOf<T>::is_i8 ? CKX_OP_CONV2D_FWD_I8 : CKX_OP_CONV2D_FWD_F16);
    for(int i = 0; i < n; ++i)
        v.push_back(std::make_unique<
                    DeviceConv2dFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<T, T, T, InOp, WeiOp, OutOp>>(
            i));
    return v;
}

// ConvolutionFwdInstances<T,T,T>::Get<NumDimSpatial>() (conv_util.hpp:288-397)
template <int NumDimSpatial, typename T, typename InOp, typename WeiOp, typename OutOp>
std::vector<std::unique_ptr<DeviceConvFwd<InOp, WeiOp, OutOp>>> GetConvNdFwdInstances()
{
    std::vector<std::unique_ptr<DeviceConvFwd<InOp, WeiOp, OutOp>>> v;
    const int n = ckx_num_instances(detail::DTypeOf<T>::is_i8 ? CKX_OP_CONV2D_FWD_I8 : CKX_OP_CONV2D_FWD_F16);
    for(int i = 0; i < n; ++i)
        v.push_back(std::make_unique<DeviceConvNDFwdMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<
                        T, T, T, InOp, WeiOp, OutOp, NumDimSpatial>>(i));
    return v;
}

// instance lists of the fused operators: one per tile configuration (the skinny GEMM instances
// are included for DeviceGemmMultipleD)
template <typename AL, typename BL, typename EL, typename Ds, typename CDEOp>
struct DeviceOperationInstanceFactory<DeviceGemmMultipleD<AL, BL, EL, half_t, half_t, Ds, half_t, element_wise::PassThrough,
                                                          element_wise::PassThrough, CDEOp>>
{
    using DeviceOp = DeviceGemmMultipleD<AL, BL, EL, half_t, half_t, Ds, half_t, element_wise::PassThrough,
                                         element_wise::PassThrough, CDEOp>;
    static std::vector<std::unique_ptr<DeviceOp>> GetInstances()
    {
        std::vector<std::unique_ptr<DeviceOp>> v;
        const int n = ckx_num_instances(CKX_OP_GEMM_F16);
        for(int i = 0; i < n; ++i)
            v.push_back(std::make_unique<DeviceGemmMultipleDMfma<AL, BL, EL, Ds, CDEOp>>(i));
        return v;
    }
};

template <typename InOp, typename WeiOp, typename OutOp>
struct DeviceOperationInstanceFactory<DeviceConvFwdBiasActivation<InOp, WeiOp, OutOp>>
{
    using DeviceOp = DeviceConvFwdBiasActivation<InOp, WeiOp, OutOp>;
    static std::vector<std::unique_ptr<DeviceOp>> GetInstances()
    {
        std::vector<std::unique_ptr<DeviceOp>> v;
        for(int i = 0, n = ckx_num_instances(CKX_OP_CONV2D_FWD_F16); i < n; ++i)
            v.push_back(std::make_unique<
                        DeviceConv2dFwdBiasActivationMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<InOp, WeiOp, OutOp>>(i));
        return v;
    }
};

template <typename InOp, typename WeiOp, typename OutOp>
struct DeviceOperationInstanceFactory<DeviceConvFwdBiasActivationAdd<InOp, WeiOp, OutOp>>
{
    using DeviceOp = DeviceConvFwdBiasActivationAdd<InOp, WeiOp, OutOp>;
    static std::vector<std::unique_ptr<DeviceOp>> GetInstances()
    {
        std::vector<std::unique_ptr<DeviceOp>> v;
        for(int i = 0, n = ckx_num_instances(CKX_OP_CONV2D_FWD_F16); i < n; ++i)
            v.push_back(std::make_unique<
                        DeviceConv2dFwdBiasActivationAddMfma_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<InOp, WeiOp, OutOp>>(i));
        return v;
    }
};

} // namespace instance
} // namespace device
} // namespace tensor_operation
} // namespace ck
