/*
 * ckx.h -- C ABI of the MI355X (gfx950) MFMA GEMM hot path.
 *
 * Every entry point replaces the launch half of one Composable Kernel device
 * operator (MakeArgumentPointer + IsSupportedArgument + Invoker::Run); the C++
 * operator classes in composable_kernel_amd/host/ckx/device_ops.hpp sit on top of
 * these calls and carry CK's own interface. All pointers are DEVICE pointers,
 * strides are in ELEMENTS, dimensions are int32 (CK's index_t, include/ck/ck.hpp:176),
 * `stream` is a hipStream_t passed as void* (NULL = default stream). Launches are
 * asynchronous; nothing is allocated, nothing is synchronised. Scratch memory, where a launch
 * can use it, is the caller's (p_workspace, see ckx_*_workspace_bytes).
 *
 * Return value: 0 on success, a negative ckx_status otherwise; the message for
 * the calling thread's last failure is returned by ckx_last_error().
 */
#ifndef CKX_H_
#define CKX_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ckx_status
{
    CKX_OK            = 0,
    CKX_UNSUPPORTED   = -1, /* IsSupportedArgument would be false */
    CKX_INVALID_VALUE = -2, /* null pointer, negative size, unknown enum */
    CKX_HIP_ERROR     = -3  /* launch failed; ckx_last_error() has hipGetErrorString */
} ckx_status;

/* tensor_layout::gemm::{RowMajor,ColumnMajor}
 * (include/ck/tensor_operation/gpu/device/tensor_layout.hpp) */
enum
{
    CKX_ROW_MAJOR = 0,
    CKX_COL_MAJOR = 1
};

/* C / Out element-wise operation applied to the accumulator before the store.
 *  PASSTHROUGH  element_wise::PassThrough (unary_element_wise_operation.hpp:13-25);
 *               int8 output keeps the low byte of the int32 accumulator.
 *  REQUANT_CK   RequantReluRequant, literal
 *               (example/14_gemm_xdl_requant_relu_requant/gemm_xdl_requant_relu_requant_int8.cpp:21-39):
 *               y = clamp(sR * relu(sG * acc), -128, 127), then truncation toward zero.
 *  REQUANT_RND  y = sat8(rint(sR * relu(sat8(rint(sG * acc))))), rint = half-to-even.
 * All arithmetic is fp32 on the exactly converted int32 accumulator, two separate
 * multiplies, no contraction. */
enum
{
    CKX_EPI_PASSTHROUGH = 0,
    CKX_EPI_REQUANT_CK  = 1,
    CKX_EPI_REQUANT_RND = 2,
    /* fp16 outputs with extra fp16 "D" operands, arithmetic in fp32, one rounding at the store:
     *  ADD_RELU           e = half(relu(acc + d0))          element_wise::AddRelu as applied by
     *                     ReferenceConvFwd_Bias_Activation (reference_conv_fwd_bias_activation.hpp:75-124)
     *  ADD_RELU_ADD       e = half(relu(acc + d0) + d1)     element_wise::AddReluAdd
     *                     (element_wise_operation.hpp:46-81, reference_conv_fwd_bias_activation_add.hpp)
     *  CSHUFFLE_ADD_RELU  e = relu(half(half(acc) + d0))    AddRelu on the C value already rounded to
     *                     fp16 (example/03_gemm_bias_relu/gemm_bias_relu_xdl_fp16.cpp:31-40,251-275) */
    CKX_EPI_ADD_RELU          = 3,
    CKX_EPI_ADD_RELU_ADD      = 4,
    CKX_EPI_CSHUFFLE_ADD_RELU = 5,
    /* int8 outputs with ONE ROW OF N fp32 REQUANT SCALES as the "D" operand (per output column of a GEMM, per output
     * channel of a conv): upstream Composable Kernel's element_wise::Activation_Mul2_Clamp<Activation>
     * (ck/tensor_operation/gpu/element/quantization_operation.hpp as shipped with ROCm; the operator is newer than
     * the reference snapshot, whose DeviceGemmMultipleD interface, device_gemm_multiple_d.hpp:14-55, it plugs into):
     *   y = float(acc); y = act(y); y = clamp(scale[n] * y, -128, 127); e = int8(y)   (truncation toward zero)
     *  MUL2_CLAMP       act = PassThrough
     *  RELU_MUL2_CLAMP  act = Relu
     * One fp32 multiply on the exactly converted accumulator (|acc| < 2^24; larger ones round to nearest even on both
     * sides); scales are finite by contract. */
    CKX_EPI_MUL2_CLAMP      = 6,
    CKX_EPI_RELU_MUL2_CLAMP = 7,
    /* fp16 GEMM outputs, fp32 arithmetic on the fp32 accumulator, one rounding at the store:
     *  BILINEAR          e = half(alpha * acc + beta * d0)        element_wise::Bilinear
     *                    (binary_element_wise_operation.hpp:93-116; example/02_gemm_bilinear/gemm_bilinear_xdl_fp16.cpp:
     *                    18-36,290-297); alpha and beta are arguments of ckx_gemm_f16_bilinear
     *  ADD_ADD_FASTGELU  e = half(fast_gelu(acc + d0 + d1))       element_wise::AddAddFastGelu
     *                    (element_wise_operation.hpp:113-140; example/04_gemm_add_add_fastgelu), with
     *                    fast_gelu(x) = x * (0.5 + 0.5 * (2 / (1 + exp(-u)) - 1)), u = 2x(0.035677 x^2 + 0.797885),
     *                    evaluated as x / (1 + exp(-u)) */
    CKX_EPI_BILINEAR         = 8,
    CKX_EPI_ADD_ADD_FASTGELU = 9
};

/* Operator families, for the instance queries below. */
enum
{
    CKX_OP_GEMM_I8           = 0,
    CKX_OP_GEMM_F16          = 1,
    CKX_OP_CONV2D_FWD_I8     = 2,
    CKX_OP_CONV2D_FWD_F16    = 3,
    CKX_OP_BATCHED_GEMM_GEMM = 4,
    CKX_OP_GEMM_SPLITK       = 5, /* instance list of the split-K GEMMs (the tile instances, both dtypes) */
    CKX_OP_GEMM_BF16         = 6,
    CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM = 7
};

#define CKX_INSTANCE_AUTO (-1)

/* ---- library ------------------------------------------------------------ */
const char* ckx_version(void);
const char* ckx_last_error(void);

/* Instance list of one operator family: what
 * DeviceOperationInstanceFactory<DeviceOp>::GetInstances() enumerates
 * (library/include/ck/library/tensor_operation_instance/gpu/gemm.hpp:233-379).
 * ckx_instance_name() is the GetTypeString() of that instance
 * (device_gemm_xdl_cshuffle.hpp:655-672). */
int ckx_num_instances(int op);
const char* ckx_instance_name(int op, int instance);

/* ---- int8 GEMM:  C = c_op(A * B), int32 accumulation ----------------------
 * Replaces DeviceGemm<..., int8_t, int8_t, int8_t, PassThrough, PassThrough, COp>
 * ::MakeArgumentPointer + Invoker::Run (device_gemm.hpp:24-41,
 * device_gemm_xdl_cshuffle.hpp:399-556) and kernel_gemm_xdl_cshuffle_v1
 * (gridwise_gemm_xdl_cshuffle_v1.hpp:32-74).
 * A is [M,K], B is [K,N], C is [M,N]; *_layout selects which stride is 1:
 *   a_layout CKX_ROW_MAJOR  "mk": A(m,k) at m*stride_a + k      CKX_COL_MAJOR "km": at k*stride_a + m
 *   b_layout CKX_COL_MAJOR  "nk": B(k,n) at n*stride_b + k      CKX_ROW_MAJOR "kn": at k*stride_b + n
 *   c_layout CKX_ROW_MAJOR only (as in the reference's instance lists
 *   device_gemm_xdl_*_{mk_kn,mk_nk,km_kn,km_nk}_mn_instance.cpp).
 * The vectorised instances (tile and skinny) need the contiguous extent of A and of B, both strides and both
 * base addresses to be whole 16-byte vectors, and report CKX_UNSUPPORTED otherwise -- the reference's
 * GemmSpecialization::Default instances (gemm_specialization.hpp:10-20). mk_nk runs on every instance; a
 * K-major operand (km / kn) on the tile instances of 64 rows and more, with the PassThrough / requant
 * epilogues. The LAST instance of every GEMM family is element-granular (any K, M, N, strides and base
 * addresses, all four layouts, every epilogue of the data type: the reference's KPadding / MNKPadding
 * instances, device_gemm_xdl_cshuffle.hpp:99-184) and CKX_INSTANCE_AUTO sends there exactly the problems
 * the vectorised instances refuse, so AUTO supports every shape. This holds for every ckx_gemm_* and
 * ckx_batched_gemm_* entry point below. */
int ckx_gemm_i8_is_supported(int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                             int32_t stride_c, int a_layout, int b_layout, int c_layout, int epilogue,
                             int instance);
int ckx_gemm_i8(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                int c_layout, int epilogue, float scale_gemm, float scale_relu, int instance,
                void* p_workspace, int64_t workspace_bytes, void* stream);
/* BaseOperator::GetWorkSpaceSize (device_base.hpp:47): bytes of device scratch with which the
 * launch may cut K into several runs (split-K: problems with too few C tiles to occupy the
 * machine). The workspace is OPTIONAL: with p_workspace == NULL, or fewer bytes than asked for,
 * the launch uses a plan that needs none. It needs no initialisation and holds nothing between
 * calls; two launches that share one workspace must not overlap. */
int64_t ckx_gemm_i8_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance);

/* ---- fp16 GEMM:  C = half(A * B), fp32 accumulation -----------------------
 * Replaces DeviceGemm<..., half_t, half_t, half_t, PassThrough x3>
 * (device_gemm.hpp:24-41; device_gemm_xdl.hpp:60-545, kernel_gemm_xdlops_v2r3). */
int ckx_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                              int32_t stride_c, int a_layout, int b_layout, int c_layout, int instance);
int ckx_gemm_f16(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                 int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                 int c_layout, int instance, void* p_workspace, int64_t workspace_bytes, void* stream);
int64_t ckx_gemm_f16_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance);

/* ---- bf16 GEMM:  C = bf16(A * B), fp32 accumulation ------------------------
 * Replaces DeviceGemm<..., bhalf_t, bhalf_t, bhalf_t, PassThrough x3> (device_gemm.hpp:24-41; the bf16
 * instances of the reference's gemm family); the conversion is round-to-nearest-even, as
 * type_convert<bhalf_t, float> (include/ck/utility/data_type.hpp:953-993). */
int ckx_gemm_bf16_is_supported(int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                               int32_t stride_c, int a_layout, int b_layout, int c_layout, int instance);
int ckx_gemm_bf16(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                  int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                  int c_layout, int instance, void* p_workspace, int64_t workspace_bytes, void* stream);
int64_t ckx_gemm_bf16_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance);

/* ---- strided batched GEMM:  C[g] = c_op(A[g] * B[g]),  g < batch ----------------
 * Replaces DeviceBatchedGemm<...>::MakeArgumentPointer(..., BatchStrideA, BatchStrideB, BatchStrideC,
 * Batch, ...) + Run (device_batched_gemm.hpp:24-45; batch offsets as ComputePtrOffsetOfStridedBatch,
 * device_batched_gemm_xdl.hpp:256-285). Batch strides are in elements. The batches share one launch:
 * the persistent workgroups walk the C tiles of all batches. Shapes as for ckx_gemm_*_is_supported on a
 * tile instance, the element-granular instance or AUTO; the C batches must not overlap and the whole A, B, C
 * extents stay below 2 GiB. On the tile instances the A / B batch strides must be multiples of 16 bytes; AUTO
 * sends other strides (up to 65535 batches) to the element-granular instance. */
int ckx_batched_gemm_is_supported(int op, int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                                  int32_t stride_c, int64_t batch_stride_a, int64_t batch_stride_b,
                                  int64_t batch_stride_c, int32_t batch, int a_layout, int b_layout, int c_layout,
                                  int epilogue, int instance);
int ckx_batched_gemm_i8(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                        int32_t stride_a, int32_t stride_b, int32_t stride_c, int64_t batch_stride_a,
                        int64_t batch_stride_b, int64_t batch_stride_c, int32_t batch, int a_layout, int b_layout,
                        int c_layout, int epilogue, float scale_gemm, float scale_relu, int instance, void* stream);
int ckx_batched_gemm_f16(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                         int32_t stride_a, int32_t stride_b, int32_t stride_c, int64_t batch_stride_a,
                         int64_t batch_stride_b, int64_t batch_stride_c, int32_t batch, int a_layout, int b_layout,
                         int c_layout, int instance, void* stream);

/* ---- split-K GEMM with a caller-chosen number of K runs ----------------------
 * Replaces DeviceGemmSplitK<...>::MakeArgumentPointer(..., KBatch) + Run (device_gemm_splitk.hpp:14-39).
 * The K extent is cut into k_batch (1..8) runs of whole 128-byte K tiles (fewer when K has fewer tiles);
 * the runs' raw int32 / fp32 accumulators go to the workspace and a second kernel adds them in run
 * order and applies the epilogue: deterministic, and for int8 bit-identical to the unsplit GEMM
 * (the reference adds with atomics into a zeroed C instead). k_batch > 1 requires a workspace of
 * ckx_gemm_splitk_workspace_bytes(op, M, N, K, k_batch) bytes (op = CKX_OP_GEMM_I8 / _F16).
 * Supported shapes are those of ckx_gemm_*_is_supported with a tile instance (or AUTO). */
int64_t ckx_gemm_splitk_workspace_bytes(int op, int32_t M, int32_t N, int32_t K, int32_t k_batch);
int ckx_gemm_i8_splitk(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                       int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                       int c_layout, int epilogue, float scale_gemm, float scale_relu, int instance,
                       int32_t k_batch, void* p_workspace, int64_t workspace_bytes, void* stream);
int ckx_gemm_f16_splitk(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                        int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                        int c_layout, int instance, int32_t k_batch, void* p_workspace, int64_t workspace_bytes,
                        void* stream);

/* ---- int8 split-K GEMM for callers that cannot allocate ----------------------
 * No counterpart in the reference. For callers that cannot call hipMalloc (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it): ckx_gemm_i8_splitk with the workspace taken from a
 * static device array of the library instead of an argument -- CKX_STATIC_WORKSPACE_BYTES per GPU, held
 * from the load of the library's code object on that GPU until the process ends. The call allocates and
 * frees nothing and synchronises nothing. A split that needs more than CKX_STATIC_WORKSPACE_BYTES
 * (ckx_gemm_splitk_workspace_bytes(CKX_OP_GEMM_I8, M, N, K, k_batch)) is refused with CKX_UNSUPPORTED.
 * Every call on one GPU uses the same array: calls that may run at the same time on one GPU (different
 * streams, or graphs replayed concurrently) race on it and must be serialised by the caller. The array needs no
 * initialisation (every slice element that is read was written by the same call). The first call on a GPU
 * looks the array's address up (hipGetSymbolAddress): make it outside a stream capture. */
#define CKX_STATIC_WORKSPACE_BYTES (32 * 1024 * 1024)
int ckx_gemm_i8_splitk_noalloc(const void* p_a, const void* p_b, void* p_c, int32_t M, int32_t N, int32_t K,
                               int32_t stride_a, int32_t stride_b, int32_t stride_c, int a_layout, int b_layout,
                               int c_layout, int epilogue, float scale_gemm, float scale_relu, int instance,
                               int32_t k_batch, void* stream);

/* ---- fp16 GEMM with fused D operands:  E = cde_op(A * B, D0 [, D1]) ----------
 * Replaces DeviceGemmMultipleD<..., Tuple<half_t[, half_t]>, half_t, PassThrough, PassThrough, CDEOp>
 * ::MakeArgumentPointer + Run (device_gemm_multiple_d.hpp:14-55) for cde_op in
 * CKX_EPI_ADD_RELU / _ADD_RELU_ADD / _CSHUFFLE_ADD_RELU / _ADD_ADD_FASTGELU (and, for the query, _BILINEAR). D0, D1 are
 * [M,N] row-major fp16 with row strides stride_d0 / stride_d1 in elements; stride 0 broadcasts one row (a bias
 * vector), as examples 03 and 04 do. p_d1 is ignored unless cde_op uses it. With a K-major operand (A column-major
 * or B row-major) these run on CKX_INSTANCE_AUTO or the element-granular instance only; an explicit tile or skinny
 * instance answers CKX_UNSUPPORTED. CKX_EPI_ADD_ADD_FASTGELU agrees with the reference's functor
 * (element_wise_operation.hpp:113-140) within rtol = atol = 1e-2, not bit for bit: the device evaluates
 * x / (1 + exp(-u)); the reference's 0.5 + 0.5 * (2 / (1 + exp(-u)) - 1) cancels to a coarse or zero factor for
 * x below about -5, where the device returns small negative values (a few fp16 subnormal steps apart). */
int ckx_gemm_f16_multiple_d_is_supported(int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                                         int32_t stride_d0, int32_t stride_d1, int32_t stride_e, int a_layout,
                                         int b_layout, int e_layout, int cde_op, int instance);
int ckx_gemm_f16_multiple_d(const void* p_a, const void* p_b, const void* p_d0, const void* p_d1, void* p_e,
                            int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b, int32_t stride_d0,
                            int32_t stride_d1, int32_t stride_e, int a_layout, int b_layout, int e_layout,
                            int cde_op, int instance, void* p_workspace, int64_t workspace_bytes, void* stream);

/* E = half(alpha * (A * B) + beta * D): DeviceGemmMultipleD<..., Tuple<half_t>, half_t, PassThrough, PassThrough,
 * Bilinear> (device_gemm_multiple_d.hpp:14-55 with binary_element_wise_operation.hpp:93-116), the operator behind
 * the reference's "gemm_bilinear" instances and profiler command (profiler/include/profile_gemm_bilinear_impl.hpp).
 * Arguments as ckx_gemm_f16_multiple_d with one D tensor; query with cde_op = CKX_EPI_BILINEAR. */
int ckx_gemm_f16_bilinear(const void* p_a, const void* p_b, const void* p_d, void* p_e, int32_t M, int32_t N,
                          int32_t K, int32_t stride_a, int32_t stride_b, int32_t stride_d, int32_t stride_e,
                          int a_layout, int b_layout, int e_layout, float alpha, float beta, int instance,
                          void* p_workspace, int64_t workspace_bytes, void* stream);

/* ---- int8 GEMM with per-column requant scales:  E = cde_op(A * B, D0), D0 = scale[N] (fp32) ----------
 * Replaces DeviceGemmMultipleD<..., int8_t, int8_t, Tuple<float>, int8_t, PassThrough, PassThrough,
 * Activation_Mul2_Clamp<Act>>::MakeArgumentPointer + Run (device_gemm_multiple_d.hpp:14-55) for cde_op in
 * CKX_EPI_MUL2_CLAMP / CKX_EPI_RELU_MUL2_CLAMP. D0 is one contiguous row of N floats, broadcast over the rows
 * (stride_d0 must be 0, as a per-channel scale is passed upstream). Every instance of the int8 GEMM family takes it
 * (tile, skinny, element-wise; K runs through the workspace) with A row-major and B column-major; with a K-major
 * operand (A column-major or B row-major) it runs on CKX_INSTANCE_AUTO or the element-granular instance only -- an
 * explicit tile or skinny instance answers CKX_UNSUPPORTED. Batches do not take it. */
int ckx_gemm_i8_multiple_d_is_supported(int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b,
                                        int32_t stride_d0, int32_t stride_e, int a_layout, int b_layout, int e_layout,
                                        int cde_op, int instance);
int ckx_gemm_i8_multiple_d(const void* p_a, const void* p_b, const void* p_d0, void* p_e, int32_t M, int32_t N,
                           int32_t K, int32_t stride_a, int32_t stride_b, int32_t stride_d0, int32_t stride_e,
                           int a_layout, int b_layout, int e_layout, int cde_op, int instance, void* p_workspace,
                           int64_t workspace_bytes, void* stream);

/* ---- conv2d forward, NHWC input / KYXC weight / NHWK output, implicit GEMM --
 * Replaces DeviceConvFwd<PassThrough, PassThrough, OutOp>::MakeArgumentPointer + Run
 * (device_conv_fwd.hpp:18-39) as implemented by
 * DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
 * (device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720).
 * The vectors of the reference interface are passed as scalars in (H, W) order:
 * in_spatial = {Hi, Wi}, filter = {Y, X}, out_spatial = {Ho, Wo}, strides = {sH, sW},
 * dilations = {dH, dW}, left pads = {pad_top, pad_left}, right pads = {pad_bottom, pad_right}.
 * The vectorised instances need C to fill whole 16-byte vectors (C % 16 for int8, C % 8 for fp16; the
 * reference: C % SrcScalarPerVector, device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:595-601) and 16-byte aligned
 * input and weight addresses. The LAST instance of both conv families is element-granular -- any C, the
 * reference's ConvolutionForwardSpecialization::OddC instances (convolution_forward_specialization.hpp:13-19)
 * -- for one, two and three spatial dimensions and every epilogue; CKX_INSTANCE_AUTO sends it the layers the
 * vectorised instances refuse. */
typedef struct ckx_conv2d_desc
{
    int32_t N, K, C;
    int32_t Hi, Wi;
    int32_t Y, X;
    int32_t Ho, Wo;
    int32_t stride_h, stride_w;
    int32_t dilation_h, dilation_w;
    int32_t pad_top, pad_left;
    int32_t pad_bottom, pad_right;
} ckx_conv2d_desc;

int ckx_conv2d_fwd_is_supported(int op, const ckx_conv2d_desc* desc, int epilogue, int instance);
int ckx_conv2d_fwd_i8(const void* p_in, const void* p_wei, void* p_out, const ckx_conv2d_desc* desc,
                      int epilogue, float scale_gemm, float scale_relu, int instance, void* p_workspace,
                      int64_t workspace_bytes, void* stream);
int ckx_conv2d_fwd_f16(const void* p_in, const void* p_wei, void* p_out, const ckx_conv2d_desc* desc,
                       int instance, void* p_workspace, int64_t workspace_bytes, void* stream);
int64_t ckx_conv2d_fwd_workspace_bytes(int op, const ckx_conv2d_desc* desc, int instance);
/* conv2d forward + bias + ReLU (+ residual add), fp16: replaces
 * DeviceConvFwdBiasActivation / DeviceConvFwdBiasActivationAdd ::MakeArgumentPointer + Run
 * (device_conv_fwd_bias_activation.hpp:18-41, device_conv_fwd_bias_activation_add.hpp).
 * p_bias is a contiguous [K] vector, p_resi has the output's NHWK layout (ignored for ADD_RELU);
 * out_op is CKX_EPI_ADD_RELU or CKX_EPI_ADD_RELU_ADD. Supported geometries are those of
 * ckx_conv2d_fwd_is_supported(CKX_OP_CONV2D_FWD_F16, desc, out_op, instance). */
int ckx_conv2d_fwd_bias_activation_f16(const void* p_in, const void* p_wei, void* p_out, const void* p_bias,
                                       const void* p_resi, const ckx_conv2d_desc* desc, int out_op, int instance,
                                       void* p_workspace, int64_t workspace_bytes, void* stream);

/* conv2d forward, int8, with one fp32 requant scale per OUTPUT CHANNEL (p_scale: K contiguous floats): out_op is
 * CKX_EPI_MUL2_CLAMP or CKX_EPI_RELU_MUL2_CLAMP (upstream's per-channel quantisation of a conv: the same functor as
 * the CDE operation of its multiple-D conv operators). Every conv instance but the streaming 1x1 one takes it (the
 * pointwise specialist for 256-byte pixels only: the scales live in registers beside the weights); supported geometries are those of
 * ckx_conv2d_fwd_is_supported(CKX_OP_CONV2D_FWD_I8, desc, out_op, instance). */
int ckx_conv2d_fwd_i8_multiple_d(const void* p_in, const void* p_wei, const void* p_scale, void* p_out,
                                 const ckx_conv2d_desc* desc, int out_op, int instance, void* p_workspace,
                                 int64_t workspace_bytes, void* stream);

/* ---- conv forward with 1, 2 or 3 spatial dimensions: NWC / NHWC / NDHWC input, KXC / KYXC / KZYXC
 * weight, NWK / NHWK / NDHWK output --------------------------------------------------------------
 * Replaces DeviceConvFwd<PassThrough, PassThrough, OutOp>::MakeArgumentPointer + Run as implemented by
 * DeviceConvNDFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K<..., NumDimSpatial>
 * (device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp:76-1046; the instances conv_util.hpp:288-397 hands out for
 * Get<1>(), Get<2>(), Get<3>()). The vectors of the reference interface arrive as arrays whose first
 * `ndim` entries are used, slowest dimension first ((D,) (H,) W). op is CKX_OP_CONV2D_FWD_I8 or _F16 (the
 * data type; the families and their instance lists are shared by every dimensionality), epilogue one of
 * PassThrough / requant for int8, PassThrough for fp16. One and two dimensions (and three with an
 * unconvolved depth axis) run as the 2-D problem; three convolved dimensions take the tile instances. */
typedef struct ckx_convnd_desc
{
    int32_t ndim;
    int32_t N, K, C;
    int32_t in[3], filter[3], out[3];
    int32_t stride[3], dilation[3], pad_left[3], pad_right[3];
} ckx_convnd_desc;

int ckx_convnd_fwd_is_supported(int op, const ckx_convnd_desc* desc, int epilogue, int instance);
int64_t ckx_convnd_fwd_workspace_bytes(int op, const ckx_convnd_desc* desc, int instance);
int ckx_convnd_fwd(int op, const void* p_in, const void* p_wei, void* p_out, const ckx_convnd_desc* desc,
                   int epilogue, float scale_gemm, float scale_relu, int instance, void* p_workspace,
                   int64_t workspace_bytes, void* stream);

/* ---- batched fused GEMM-GEMM, fp16:  C[g] = half( half(A[g]*B0[g]) * B1[g] ) --
 * The reference snapshot has no such operator; the surface is upstream's
 * DeviceBatchedGemmGemm::MakeArgumentPointer (device_batched_gemm_gemm.hpp:15-56 of
 * later Composable Kernel releases), with the batch offsets of
 * kernel_batched_gemm_xdlops_v2r3 (device_batched_gemm_xdl.hpp:49-117).
 * Layout "gmk_gnk_gno_gmo": A [G,M,K] row-major, B0 column-major (memory [G,N,K]),
 * B1 [G,N,O] row-major, C [G,M,O] row-major. The [M,N] intermediate stays on chip.
 * Limits: K, O <= 128; K, O and the A / B0 / B1 strides multiples of 8 elements; B0 and B1 of ONE batch below 2 GiB each
 * (N * stride * 2 bytes: the kernels address a batch's rows through 32-bit buffer offsets). */
int ckx_batched_gemm_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t O, int32_t batch,
                                           int32_t stride_a, int32_t stride_b0, int32_t stride_b1,
                                           int32_t stride_c, int64_t batch_stride_a,
                                           int64_t batch_stride_b0, int64_t batch_stride_b1,
                                           int64_t batch_stride_c, int instance);
int ckx_batched_gemm_gemm_f16(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, int32_t M,
                              int32_t N, int32_t K, int32_t O, int32_t batch, int32_t stride_a,
                              int32_t stride_b0, int32_t stride_b1, int32_t stride_c,
                              int64_t batch_stride_a, int64_t batch_stride_b0, int64_t batch_stride_b1,
                              int64_t batch_stride_c, int instance, void* stream);

/* ---- batched fused GEMM + softmax + GEMM ("attention"), fp16 ------------------
 *   C[g] = half( half(softmax_n(mask(acc0_scale * (A[g] * B0[g])))) * B1[g] )
 * The surface is upstream's DeviceBatchedGemmSoftmaxGemm::MakeArgumentPointer
 * (device_batched_gemm_softmax_gemm.hpp:29-62 of later Composable Kernel releases) with
 * Acc0ElementwiseOperation = Scale{acc0_scale}, every other functor PassThrough, and the class's
 * MaskOutUpperTriangle parameter as an argument (scores with n > m count as -infinity). The pieces
 * are the reference's: ReferenceBatchedGemm (reference_batched_gemm.hpp:56-88) and ReferenceSoftmax
 * over n in fp32 (reference_softmax.hpp:61-113: exp(x - max) / sum). Layouts and limits as for
 * ckx_batched_gemm_gemm_f16; neither the scores nor the probabilities leave the chip. The softmax
 * is computed in one pass with a running maximum, so the probabilities are rounded to fp16 BEFORE
 * the division by the row sum (the reference rounds after it): results agree within fp16 rounding
 * of the probabilities, not bit for bit. N == 0 gives C = 0. */
int ckx_batched_gemm_softmax_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t O, int32_t batch,
                                                   int32_t stride_a, int32_t stride_b0, int32_t stride_b1,
                                                   int32_t stride_c, int64_t batch_stride_a,
                                                   int64_t batch_stride_b0, int64_t batch_stride_b1,
                                                   int64_t batch_stride_c, float acc0_scale,
                                                   int mask_out_upper_triangle, int instance);
int ckx_batched_gemm_softmax_gemm_f16(const void* p_a, const void* p_b0, const void* p_b1, void* p_c, int32_t M,
                                      int32_t N, int32_t K, int32_t O, int32_t batch, int32_t stride_a,
                                      int32_t stride_b0, int32_t stride_b1, int32_t stride_c,
                                      int64_t batch_stride_a, int64_t batch_stride_b0, int64_t batch_stride_b1,
                                      int64_t batch_stride_c, float acc0_scale, int mask_out_upper_triangle,
                                      int instance, void* stream);

/* ---- what a launch would use (pure host) ---------------------------------------
 * No counterpart in the reference, whose callers time every instance themselves (profile_gemm_impl.hpp:133-209):
 * the instance and the number of K runs that ckx_gemm_* / ckx_batched_gemm_* (op = CKX_OP_GEMM_I8 / _F16 / _BF16) or
 * ckx_conv2d_fwd_* would use for this problem with `workspace_bytes` of 16-byte aligned workspace (0: none).
 * *instance is in / out: CKX_INSTANCE_AUTO asks for the automatic choice, an instance index for that instance's K
 * split. Operand addresses are taken to be 16-byte aligned (a launch sends misaligned ones to the element-granular
 * instance). The automatic choice is a cost model; tests/golden/planner_audit.json holds what it was measured against. */
int ckx_gemm_plan(int op, int32_t M, int32_t N, int32_t K, int32_t stride_a, int32_t stride_b, int32_t stride_c,
                  int a_layout, int b_layout, int c_layout, int epilogue, int32_t batch, int64_t workspace_bytes,
                  int* instance, int* k_runs);
int ckx_conv2d_fwd_plan(int op, const ckx_conv2d_desc* desc, int epilogue, int64_t workspace_bytes, int* instance,
                        int* k_runs);
/* Tuning / test knob: force `k_runs` K runs (0: automatic) wherever a problem and its workspace allow the split;
 * returns the value in force before. The initial value is the environment variable CKX_KSPLIT, read once. */
int ckx_set_forced_k_runs(int k_runs);
/* Tuning / test knob: the 256 x 256 tile instance has two kernel bodies for dense K-contiguous GEMMs with a plain
 * epilogue -- eight waves (two per SIMD) and four waves (one per SIMD, 128 x 128 wave tiles), bit-identical results.
 * 4 or 8 forces one of them wherever both apply, 0 lets the library choose by problem size; returns the value in force
 * before. The initial value is the environment variable CKX_BIG_TILE_WAVES, read once. */
int ckx_set_big_tile_waves(int waves);

/* ---- timing helper --------------------------------------------------------
 * launch_and_time_kernel (include/ck/device_utility/kernel_launch.hpp:13-74):
 * `fn(user)` is called n_warmup times untimed, then n_repeat times between two
 * HIP events recorded on `stream`; the mean milliseconds per call is stored in
 * *ms. fn must enqueue its work on `stream` and return 0. */
typedef int (*ckx_launch_fn)(void* user);
int ckx_time_launches(ckx_launch_fn fn, void* user, int n_warmup, int n_repeat, void* stream, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* CKX_H_ */
