// Tile GEMM for gfx950 (MI355X): C[M,N] = epilogue(A[M,K] * B[N,K]^T), both operands
// K-contiguous ("mk_nk_mn": A row-major, B column-major, C row-major), with an optional
// implicit-im2col A operand for NHWC conv2d forward.
//
// Takes the place of kernel_gemm_xdl_cshuffle_v1 / kernel_gemm_xdlops_v2r3 of the
// reference (include/ck/tensor_operation/gpu/grid/gridwise_gemm_xdl_cshuffle_v1.hpp:32-74,
// gridwise_gemm_xdlops_v2r3.hpp:30-72). Nothing of their structure is kept:
//
//  * byte-generic K tiling: one K tile is 128 BYTES of every row (128 int8 / 64 fp16), so a
//    row of a staged tile is eight 16-byte chunks for either dtype, and one MFMA k-step
//    (16x16x64 i8 or 16x16x32 f16) consumes four of them: lane l reads chunk 4*ks + l/16 of
//    row l%16 with a single ds_read_b128.
//  * global -> LDS staging is direct (buffer_load_dwordx4 ... lds): a wave instruction
//    deposits 64 x 16 B = 8 rows x 8 chunks contiguously, and each lane picks WHICH global
//    chunk lands in its slot, which is how the XOR swizzle and the B row permutation are
//    applied for free. Out-of-range rows / K tail / conv padding use an out-of-range buffer
//    offset, which the hardware turns into zeros.
//  * NST LDS stages in a ring, one barrier per K tile; the kernel is persistent over work units
//    (C tile x K run x batch) and the loads run ahead of the MFMAs across unit boundaries.
//  * MFMA is issued as D^T = B_frag x A_frag, so a lane ends up owning, for one row m, the
//    accumulators of 4 consecutive columns per MFMA tile; the B rows of a 64-column group
//    are permuted in LDS so that the 4 tiles of the group give the lane 16 CONSECUTIVE
//    columns. The epilogue (requant, ReLU, saturation, conversion) runs on registers and
//    each lane stores 16 contiguous outputs: no trip through LDS.
//  * optional extras of a launch: a K split with raw accumulators in a caller workspace and a
//    second pass (splitk_reduce_kernel), fp16 add / ReLU epilogues with D operands, a strided batch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include <utility>

namespace ckx {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

enum
{
    DT_I8   = 0,
    DT_F16  = 1,
    DT_BF16 = 2 // bfloat16 operands and output, fp32 accumulation, one round-to-nearest-even conversion
};

enum
{
    EPI_PASSTHROUGH = 0,
    EPI_REQUANT_CK  = 1,
    EPI_REQUANT_RND = 2,
    // fp16 outputs with extra "D" operands (bias row / residual tensor), all arithmetic in fp32:
    EPI_ADD_RELU          = 3, // e = half(relu(acc + d0))
    EPI_ADD_RELU_ADD      = 4, // e = half(relu(acc + d0) + d1)
    EPI_CSHUFFLE_ADD_RELU = 5, // e = relu(half(half(acc) + d0)): C rounded to fp16 before the functor
    // int8 outputs with a per-column fp32 requant scale as the "D" operand (d0 = scale[N]): upstream's
    // element_wise::Activation_Mul2_Clamp<PassThrough / Relu>, e = int8(clamp(scale[n] * act(float(acc)), -128, 127))
    EPI_MUL2_CLAMP      = 6,
    EPI_RELU_MUL2_CLAMP = 7,
    // fp16 outputs again (GEMM only; the two scalars travel in scale_gemm / scale_relu):
    EPI_BILINEAR         = 8, // e = half(alpha * acc + beta * d0)
    EPI_ADD_ADD_FASTGELU = 9  // e = half(fast_gelu(acc + d0 + d1))
};
__host__ __device__ constexpr bool epi_per_column_scale(int epi) { return epi == EPI_MUL2_CLAMP || epi == EPI_RELU_MUL2_CLAMP; }
// fp16 epilogues that read a second D tensor
__host__ __device__ constexpr bool epi_has_d1(int epi) { return epi == EPI_ADD_RELU_ADD || epi == EPI_ADD_ADD_FASTGELU; }

// C tile stores: plain, or streaming (non-temporal) when the output is too large to be worth
// keeping in L2: dirty lines of a streamed output otherwise queue up behind the write-back
// and the store acknowledgements stall the K pipeline of the next tile.
// (Written as inline assembly: two stores that differ only in the non-temporal hint get merged
// into one plain store by the optimiser.)
template <typename V>
__device__ __forceinline__ void store_vec(V* ptr, V val, bool nt)
{
    static_assert(sizeof(V) == 16, "16-byte vector store");
    if(nt)
        asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(ptr), "v"(val) : "memory");
    else
        *ptr = val;
}

// q = n / d for 0 <= n < 2^31 (include/ck/utility/magic_division.hpp:28-54,132-137)
struct MagicDiv
{
    uint32_t mul;
    uint32_t shift;
    uint32_t d;
};

__device__ __forceinline__ uint32_t magic_div(uint32_t n, const MagicDiv& m)
{
    return (__umulhi(n, m.mul) + n) >> m.shift;
}

// Geometry of the implicit-GEMM view of a conv2d forward
// (device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:224-301 in closed form):
//   row m -> (n, ho, wo), k -> (y, x, c) with c fastest.
struct ConvGeom
{
    int Hi, Wi, C;
    int sH, sW, dH, dW, pT, pL;
    MagicDiv div_howo; // Ho*Wo
    MagicDiv div_wo;   // Wo
    MagicDiv div_xc;   // X*C
    MagicDiv div_c;    // C
    // three spatial dimensions (device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp, NumDimSpatial == 3):
    //   row m -> (n, do, ho, wo), k -> (z, y, x, c); depth extent, stride, dilation, front padding
    int Di, sD, dD, pF;
    MagicDiv div_dhowo; // Do*Ho*Wo
    MagicDiv div_yxc;   // Y*X*C
};

struct GemmArgs
{
    const void* a;
    const void* b;
    void* c;
    int M, N, K;
    int lda, ldb, ldc;      // elements
    uint32_t a_bytes;       // extent of the A / B allocations seen by the buffer resource
    uint32_t b_bytes;
    int tiles_m, tiles_n;
    int epi;
    float scale_gemm, scale_relu;
    int nt_store; // stream the C tile past L2 (large outputs)
    // split-K: the K tiles of every C tile are cut into `ksplit` runs of `nk_per` K tiles; run s
    // writes its raw accumulators to slice s of the workspace ([ksplit][M][N] int32 / fp32) and a
    // second kernel sums the slices and applies the epilogue. ksplit == 1: no workspace.
    int ksplit, nk_per;
    void* ws;
    // fp16 "D" operands of the fused add epilogues, [M,N] row-major with row strides ldd0 / ldd1
    // in elements (0: one row broadcast over M, i.e. a bias vector)
    const void* d0;
    const void* d1;
    int ldd0, ldd1;
    // strided batch (DeviceBatchedGemm): batch g reads A + g*bsa, B + g*bsb, writes C + g*bsc
    // (element strides); 0 or 1 = a single GEMM. The byte extents a_bytes / b_bytes span all batches.
    int batch;
    long bsa, bsb, bsc;
    ConvGeom cv;
};

constexpr uint32_t kOutOfRange = 0x80000000u;

// LDS row (position in the staged B tile) -> column of the tile. Within a 64-column group,
// LDS row 16*t + j (MFMA tile t, MFMA row j) holds column 16*(j/4) + 4*t + j%4.
__device__ __forceinline__ uint32_t b_row_to_col(uint32_t r)
{
    return (r & ~63u) | (((r & 15u) >> 2) << 4) | (((r >> 4) & 3u) << 2) | (r & 3u);
}

// Workgroup id -> tile. Workgroups are dealt round-robin to the 8 XCDs, each with a private
// L2: first make the ids that land on one XCD contiguous, then sweep tiles in groups of 8
// tile-rows, column by column, so that the tiles resident on an XCD share few A/B panels.
// (BlockToCTileMap_M00_N0_M01Adapt, block_to_ctile_map.hpp:112-173, is the reference's
// single-L2 analogue; the order is not observable in the results.)
// With batches the ids are made contiguous over the tiles of ALL batches (id = batch * tiles + tile), so that an
// XCD works on whole batches: 16 batches of 4 x 4 tiles put 2 batches = 16 operand panels on an XCD, where a
// per-batch shuffle would give it two tiles of every batch, about 48 panels (fp16 16 x 1024^3: 39.2 -> 35 us).
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int nbatch, int& batch, int& tm, int& tn)
{
    const int nb    = tiles_m * tiles_n;
    const int nall  = nb * nbatch;
    const int xcd   = bid & 7;
    const int local = bid >> 3;
    const int q = nall >> 3, r = nall & 7;
    const int gid = xcd * q + (xcd < r ? xcd : r) + local;
    batch         = gid / nb;
    const int id  = gid - batch * nb;
    constexpr int GM    = 8;
    const int per_group = GM * tiles_n;
    const int grp       = id / per_group;
    const int first_m   = grp * GM;
    const int gsz       = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int in        = id - grp * per_group;
    tm                  = first_m + in % gsz;
    tn                  = in / gsz;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>)
{
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// LDS fragment reads as inline assembly. The compiler orders every LDS read it knows about after ALL
// outstanding direct global->LDS loads (s_waitcnt vmcnt(0): it cannot tell which stage they fill),
// which would hold the first reads of a K tile until the prefetch of the tile after next has landed.
// Reads it does not know about are not counted in lgkmcnt either: the kernel waits for them itself
// (s_waitcnt lgkmcnt(0) followed by a scheduling barrier) before the first instruction that uses them.
// (No "memory" clobber: that alone makes the statement a possible LDS access and brings the wait back.
// volatile keeps the statements in program order among themselves and with the loads and stores.)
template <int IMM>
__device__ __forceinline__ i32x4 lds_read_b128(uint32_t addr)
{
    static_assert(IMM >= 0 && IMM < 65536, "16-bit offset field");
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
    return v;
}
// transposing reads (gfx950): 16 lanes x 8 bytes = a 4 x 16 block of 16-bit (8 x 16 of 8-bit) elements,
// each lane ends up with one column of it
template <int ES, int IMM>
__device__ __forceinline__ i32x2 lds_read_tr_b64(uint32_t addr)
{
    static_assert(IMM >= 0 && IMM < 65536, "16-bit offset field");
    i32x2 v;
    if constexpr(ES == 2)
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
    else
        asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(IMM));
    return v;
}

// ---------------------------------------------------------------- epilogues
// All in fp32 on the exactly converted int32 accumulator; the two multiplies are separate
// roundings (the translation unit is built with -ffp-contract=off). v_med3_f32 does a
// two-sided clamp in one instruction; "clamp to [-128,127] then ReLU" is the single clamp
// to [0,127]. Scales are finite by contract, so no NaN reaches the min/max/med3 forms.
__device__ __forceinline__ int requant_ck(int acc, float sg, float sr)
{
    float x = (float)acc;
    float g = sg * x;
    float r = __builtin_fmaxf(g, 0.0f);
    float q = sr * r;
    float y = __builtin_amdgcn_fmed3f(q, -128.0f, 127.0f);
    return (int)y; // toward zero
}

__device__ __forceinline__ int requant_rnd(int acc, float sg, float sr)
{
    float x = (float)acc;
    float t = __builtin_rintf(sg * x);
    float r = __builtin_amdgcn_fmed3f(t, 0.0f, 127.0f);
    float u = __builtin_rintf(sr * r);
    u       = __builtin_amdgcn_fmed3f(u, -128.0f, 127.0f);
    return (int)u;
}

// Activation_Mul2_Clamp: the activation runs on the converted accumulator (ReLU of an integer-valued float is the
// float of max(acc, 0)), one fp32 multiply by the column's scale, clamp, truncation toward zero (type_convert<int8_t>)
__device__ __forceinline__ int mul2_clamp(int acc, float scale, bool relu)
{
    const float x = (float)(relu && acc < 0 ? 0 : acc);
    const float y = __builtin_amdgcn_fmed3f(scale * x, -128.0f, 127.0f);
    return (int)y;
}

template <int EPI>
__device__ __forceinline__ int epilogue_i8(int acc, float sg, float sr)
{
    if constexpr(EPI == EPI_REQUANT_CK)
        return requant_ck(acc, sg, sr);
    else if constexpr(EPI == EPI_REQUANT_RND)
        return requant_rnd(acc, sg, sr);
    else
        return acc;
}

// low bytes of four ints -> one dword (b0 in bits 0-7): three byte permutes
__device__ __forceinline__ int pack4_low_bytes(int b0, int b1, int b2, int b3)
{
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b1, (uint32_t)b0, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)b3, (uint32_t)b2, 0x0c0c0400u);
    return (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// ---- the rounded requant epilogue through a 256-byte table ---------------------------------------------------
// y = sat8(rint(sR * relu(sat8(rint(sG * acc))))) has an integer in [0, 127] in the middle: r = clamp(rint(sG * acc),
// 0, 127). Everything after r is a function of 128 values, tabulated once per workgroup WITH THE SAME fp32 operations
// (requant_tail), and r itself comes out of one instruction: v_cvt_pk_u8_f32 rounds to nearest even and saturates to
// [0, 255] (entries 128 .. 255 of the table repeat entry 127), and it ORs the byte into a third operand -- the
// 256-byte-aligned LDS address of the table -- so that its result IS the address of the table entry. Per value: int ->
// float, multiply, convert-and-address, one LDS byte read; the eight VALU operations of requant_rnd become three.
// Bit-identical to requant_rnd for finite scales (the exhaustive accumulator sweep of the GPU tests drives both).
__device__ __forceinline__ int requant_tail(int r_index, float sr)
{
    const float r = (float)(r_index < 127 ? r_index : 127);
    float u       = __builtin_rintf(sr * r);
    u             = __builtin_amdgcn_fmed3f(u, -128.0f, 127.0f);
    return (int)u;
}
// fills the table at LDS byte address lut_lds (256-byte aligned); the caller provides the barrier before the first use
__device__ __forceinline__ void requant_lut_fill(uint8_t* lut, float sr, int tid, int nthreads)
{
    for(int i = tid; i < 256; i += nthreads)
        lut[i] = (uint8_t)requant_tail(i, sr);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // written before this wave reaches the barrier
}
__device__ __forceinline__ int lds_read_u8(uint32_t addr)
{
    int v;
    asm volatile("ds_read_u8 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
// 4 * NQ accumulators -> their 4 * NQ requantised bytes b[], through the table (the reads are inline assembly, waited
// for here: see lds_read_b128; LDS reads return in order, so whatever else the wave has in flight is complete too)
template <int NQ>
__device__ __forceinline__ void requant_lut(const i32x4 (&v)[NQ], float sg, uint32_t lut_lds, int (&b)[4 * NQ])
{
#pragma unroll
    for(int t = 0; t < NQ; ++t)
#pragma unroll
        for(int j = 0; j < 4; ++j)
            b[t * 4 + j] = lds_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(sg * (float)v[t][j], 0u, lut_lds));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// 16 consecutive int8 outputs of one row, rounded requant through the table
__device__ __forceinline__ void store_row16_i8_lut(int8_t* crow, int n0, int N, bool vec_ok, const i32x4 (&v)[4], float sg,
                                                   uint32_t lut_lds, bool nt)
{
    int b[16];
    requant_lut<4>(v, sg, lut_lds, b);
    if(vec_ok && n0 + 16 <= N)
    {
        i32x4 pk;
#pragma unroll
        for(int w = 0; w < 4; ++w)
            pk[w] = pack4_low_bytes(b[4 * w], b[4 * w + 1], b[4 * w + 2], b[4 * w + 3]);
        store_vec(reinterpret_cast<i32x4*>(crow + n0), pk, nt);
    }
    else
    {
#pragma unroll
        for(int e = 0; e < 16; ++e)
            if(n0 + e < N)
                crow[n0 + e] = (int8_t)b[e];
    }
}

// 16 consecutive int8 outputs of one row
template <int EPI>
__device__ __forceinline__ void store_row16_i8(int8_t* crow, int n0, int N, bool vec_ok, const i32x4 (&v)[4],
                                               float sg, float sr, bool nt = false)
{
    int b[16];
#pragma unroll
    for(int t = 0; t < 4; ++t)
#pragma unroll
        for(int j = 0; j < 4; ++j)
            b[t * 4 + j] = epilogue_i8<EPI>(v[t][j], sg, sr);
    if(vec_ok && n0 + 16 <= N)
    {
        i32x4 pk;
#pragma unroll
        for(int w = 0; w < 4; ++w)
            pk[w] = pack4_low_bytes(b[4 * w], b[4 * w + 1], b[4 * w + 2], b[4 * w + 3]);
        store_vec(reinterpret_cast<i32x4*>(crow + n0), pk, nt);
    }
    else
    {
#pragma unroll
        for(int e = 0; e < 16; ++e)
            if(n0 + e < N)
                crow[n0 + e] = (int8_t)b[e];
    }
}

// 16 consecutive int8 outputs of one row under per-column scales sc[0..15] (columns n0 .. n0 + 15)
__device__ __forceinline__ void store_row16_i8_cols(int8_t* crow, int n0, int N, bool vec_ok, const i32x4 (&v)[4],
                                                    const float (&sc)[16], bool relu, bool nt = false)
{
    int b[16];
#pragma unroll
    for(int t = 0; t < 4; ++t)
#pragma unroll
        for(int j = 0; j < 4; ++j)
            b[t * 4 + j] = mul2_clamp(v[t][j], sc[t * 4 + j], relu);
    if(vec_ok && n0 + 16 <= N)
    {
        i32x4 pk;
#pragma unroll
        for(int w = 0; w < 4; ++w)
            pk[w] = pack4_low_bytes(b[4 * w], b[4 * w + 1], b[4 * w + 2], b[4 * w + 3]);
        store_vec(reinterpret_cast<i32x4*>(crow + n0), pk, nt);
    }
    else
    {
#pragma unroll
        for(int e = 0; e < 16; ++e)
            if(n0 + e < N)
                crow[n0 + e] = (int8_t)b[e];
    }
}

// the 16 scales of columns n0 .. n0 + 15 (zeros past N: a bounds-checked buffer read, no alignment beyond a float's)
__device__ __forceinline__ void load_col_scales(const __amdgpu_buffer_rsrc_t& rs, int n0, float (&sc)[16])
{
#pragma unroll
    for(int e = 0; e < 16; ++e)
        sc[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, (n0 + e) * 4, 0, 0));
}

// The fused add epilogues of the fp16 path (element-wise functors AddRelu / AddReluAdd of
// include/ck/tensor_operation/gpu/element/{binary_,}element_wise_operation.hpp as the host
// references apply them: reference_conv_fwd_bias_activation[_add].hpp on the fp32 accumulator,
// example/03_gemm_bias_relu on the accumulator already rounded to fp16).
// EXT = false leaves the scaled / GELU modes out of the generated code (callers that have already branched on them).
// fast_gelu(x) = x / (1 + exp(-2x(0.035677 x^2 + 0.797885))), the closed form of the reference's
// 0.5 + 0.5 * (2 / (1 + emu) - 1) (element_wise_operation.hpp:127-133), the quotient through v_rcp_f32;
// x -> -inf gives exp -> +inf, a reciprocal of 0 and -0. Not bit for bit the reference's functor: its form cancels to a
// coarse or zero factor for x below about -5, where this one returns small negative values (a few fp16 subnormal
// steps apart) -- parity with it is by tolerance (rtol = atol = 1e-2).
template <bool EXT = true>
__device__ __forceinline__ float epi_f16_value(int mode, float acc, float d0, float d1, float alpha = 1.0f,
                                               float beta = 1.0f)
{
    if constexpr(EXT)
    {
        if(mode == EPI_BILINEAR)
            return alpha * acc + beta * d0;
        if(mode == EPI_ADD_ADD_FASTGELU)
        {
            const float x = acc + d0 + d1;
            const float u = 2.0f * x * (0.035677f * x * x + 0.797885f);
            return x * __builtin_amdgcn_rcpf(1.0f + __expf(-u)); // (v_rcp_f32: one ulp of fp32)
        }
    }
    if(mode == EPI_CSHUFFLE_ADD_RELU)
    {
        const float x = (float)(_Float16)((float)(_Float16)acc + d0);
        return x > 0.0f ? x : 0.0f;
    }
    const float a = acc + d0;
    const float b = a > 0.0f ? a : 0.0f;
    return mode == EPI_ADD_RELU_ADD ? b + d1 : b;
}

// How a copy of the fused epilogue knows its functor: FunctorIs<M> fixes it when the copy is compiled (nothing of the
// other functors is left in it); FunctorOf<D1, EXT> fixes the operand count and the family only and reads the functor
// from the arguments, one copy serving several.
template <int M>
struct FunctorIs
{
    static constexpr bool has_d1 = epi_has_d1(M), ext = M >= EPI_BILINEAR;
    __device__ static constexpr int mode(const GemmArgs&) { return M; }
};
template <bool D1, bool EXT, bool CONV = false>
struct FunctorOf
{
    static constexpr bool has_d1 = D1, ext = EXT;
    // (with a second D tensor the only extended functor is the GELU one, without it the bilinear one)
    __device__ static int mode(const GemmArgs& p)
    {
        // (and two of the plain functors take one D tensor, of which the conv operators use add + ReLU only)
        return EXT ? (D1 ? (int)EPI_ADD_ADD_FASTGELU : (int)EPI_BILINEAR)
               : D1 ? (int)EPI_ADD_RELU_ADD
               : CONV ? (int)EPI_ADD_RELU
                      : p.epi;
    }
};

// 16 consecutive fp16 outputs of one row with D operands; d0row / d1row point at column 0 of the
// row's D values (d1row may be null)
__device__ __forceinline__ void store_row16_f16_fused(_Float16* crow, int n0, int N, bool vec_ok, f32x4 (&v)[4],
                                                      int mode, const _Float16* d0row, const _Float16* d1row,
                                                      bool dvec_ok, bool nt, float alpha, float beta);

// T = _Float16 or __bf16
template <typename T>
__device__ __forceinline__ void store_row16_f16(T* crow, int n0, int N, bool vec_ok, const f32x4 (&v)[4],
                                                bool nt = false)
{
    typedef T tx8 __attribute__((ext_vector_type(8)));
    if(vec_ok && n0 + 16 <= N)
    {
        tx8 lo, hi;
#pragma unroll
        for(int j = 0; j < 4; ++j)
        {
            lo[j]     = (T)v[0][j];
            lo[4 + j] = (T)v[1][j];
            hi[j]     = (T)v[2][j];
            hi[4 + j] = (T)v[3][j];
        }
        store_vec(reinterpret_cast<tx8*>(crow + n0), lo, nt);
        store_vec(reinterpret_cast<tx8*>(crow + n0 + 8), hi, nt);
    }
    else
    {
#pragma unroll
        for(int t = 0; t < 4; ++t)
#pragma unroll
            for(int j = 0; j < 4; ++j)
                if(n0 + t * 4 + j < N)
                    crow[n0 + t * 4 + j] = (T)v[t][j];
    }
}

__device__ __forceinline__ void store_row16_f16_fused(_Float16* crow, int n0, int N, bool vec_ok, f32x4 (&v)[4],
                                                      int mode, const _Float16* d0row, const _Float16* d1row,
                                                      bool dvec_ok, bool nt, float alpha, float beta)
{
    const bool has_d1 = epi_has_d1(mode);
    if(dvec_ok && n0 + 16 <= N)
    {
        const f16x8 z   = {0, 0, 0, 0, 0, 0, 0, 0};
        const f16x8 b_lo = *reinterpret_cast<const f16x8*>(d0row + n0);
        const f16x8 b_hi = *reinterpret_cast<const f16x8*>(d0row + n0 + 8);
        const f16x8 r_lo = has_d1 ? *reinterpret_cast<const f16x8*>(d1row + n0) : z;
        const f16x8 r_hi = has_d1 ? *reinterpret_cast<const f16x8*>(d1row + n0 + 8) : z;
#pragma unroll
        for(int t = 0; t < 4; ++t)
#pragma unroll
            for(int j = 0; j < 4; ++j)
            {
                const int e = t * 4 + j;
                v[t][j]     = epi_f16_value(mode, v[t][j], (float)(e < 8 ? b_lo[e] : b_hi[e - 8]),
                                            (float)(e < 8 ? r_lo[e] : r_hi[e - 8]), alpha, beta);
            }
    }
    else
    {
#pragma unroll
        for(int t = 0; t < 4; ++t)
#pragma unroll
            for(int j = 0; j < 4; ++j)
            {
                const int n = n0 + t * 4 + j;
                if(n < N)
                    v[t][j] = epi_f16_value(mode, v[t][j], (float)d0row[n], has_d1 ? (float)d1row[n] : 0.0f, alpha, beta);
            }
    }
    store_row16_f16(crow, n0, N, vec_ok, v, nt);
}

// ------------------------------------------------------------------- kernel
// BKB   bytes of every row staged per K tile (128)
// NST   LDS stages: the loads of K tile k + NST are issued while tile k is multiplied (2: big tiles
//       that fill the LDS; 4: small tiles of latency-bound problems)
// The kernel is PERSISTENT: workgroup b works on tiles b, b + gridDim.x, ... and the K-tile
// pipeline runs straight across tile boundaries, so the first loads of the next tile are in
// flight under the last MFMAs, the epilogue arithmetic and the C stores of the current one.
//
// TA / TB: the operand is stored K-MAJOR (A column-major "km": element (m,k) at k*lda + m; B row-major
// "kn": element (k,n) at k*ldb + n). Its staged tile is then [k row][m or n], 16-byte chunks of 8 fp16 /
// 16 int8 consecutive m (n), and the MFMA fragments come out of LDS through the transposing reads
// ds_read_b64_tr_b16 / _b8: within 16 lanes, lane 4e+j (b16; 2e+j for b8) points at 4 (8) consecutive
// elements of k row e, and lane i receives element i of every one of the 4 (8) rows -- four (eight)
// consecutive k of ONE m, i.e. half an MFMA operand. A K-major B tile keeps its columns in natural
// order (the transposing read has no room for the column permutation of the K-contiguous path), and
// the epilogue moves accumulators between the four 16-lane rows instead (transpose_acc).
//
// FUSED (fp16): the variant with the add / ReLU epilogues and their D operands. A kernel of its own: the
// D values of that epilogue take registers (256 x 128: 171 VGPRs against 146; im2col 194 against 150) that
// launches which never run it need not pay for. Its K loop is the plain one as long as the epilogue awaits
// its D loads explicitly (see d_values_landed there).
template <int DT, int BM, int BN, int WM, int WN, int BKB, int NST, int IM2COL, bool TA = false, bool TB = false,
          bool FUSED = false>
struct GemmTile
{
    static constexpr int NW      = WM * WN;
    static constexpr int NT      = NW * 64;
    static constexpr int ES      = DT == DT_I8 ? 1 : 2;
    static constexpr int CPR     = BKB / 16;  // 16-byte chunks per staged row
    static constexpr int RPI     = 64 / CPR;  // rows covered by one wave-wide direct load
    static constexpr int KSTEPS  = BKB / 64;  // MFMA k-steps per K tile
    static constexpr int WTM     = BM / WM;
    static constexpr int WTN     = BN / WN;
    static constexpr int MT      = WTM / 16;
    static constexpr int NG      = WTN / 64;
    // MFMAs written out with the accumulator tied to itself. Left to the compiler, the im2col kernels with the D
    // epilogues on 256-row tiles of at most 128 columns let the accumulators wander (results into freed fragment
    // registers) and copy all of them back in place at the end of EVERY K iteration, behind the last MFMA (bias + ReLU
    // on a 512-channel 3x3 layer: 68.7 us against 61.0 plain; tied: 62.8). The compiler does not see such an MFMA:
    // what it orders by itself between a matrix instruction and the vector instructions around it is written out where
    // the accumulators change hands (acc_handover).
    static constexpr bool TIED_MFMA = FUSED && DT == DT_F16 && IM2COL != 0 && BM == 256 && BN <= 128;
    static constexpr int A_TILE  = BM * BKB;
    static constexpr int B_TILE  = BN * BKB;
    static constexpr int STAGE   = A_TILE + B_TILE;
    // table of the rounded requant epilogue, after the stages -- unless its 256 bytes would cost a co-resident
    // workgroup (two 256 x 64 workgroups fill the 160 KB exactly: that instance keeps the arithmetic epilogue)
    static constexpr int LDS_CU  = 160 * 1024;
    static constexpr bool USE_LUT = DT == DT_I8 && LDS_CU / (NST * STAGE) == LDS_CU / (NST * STAGE + 256);
    static constexpr int LUT     = USE_LUT ? 256 : 0;
    static constexpr int LDS     = NST * STAGE + LUT;
    static constexpr int NLA     = BM * CPR / NT; // 16-byte loads per thread and K tile, A
    static constexpr int NLB     = BN * CPR / NT;
    static constexpr int LPT     = NLA + NLB;
    static_assert(BKB == 128 && KSTEPS == 2, "pipeline written for 128-byte K tiles");
    static_assert(NST >= 2 && (NST - 2) * LPT < 64, "vmcnt is a 6-bit counter");
    static_assert(WTM % 16 == 0 && WTN % 64 == 0, "wave tile must be 16k x 64k");
    static_assert((BM * CPR) % NT == 0 && (BN * CPR) % NT == 0, "tile rows must split over the waves");

    static_assert(IM2COL >= 0 && IM2COL <= 2 && !(IM2COL != 0 && (TA || TB)), "the im2col view (1: two spatial dimensions, 2: three) is K-contiguous");
    static_assert(!FUSED || ((DT == DT_F16 || DT == DT_I8) && !TA && !TB),
                  "D-operand epilogues (fp16: add / ReLU functors; int8: per-column requant scales): K-contiguous operands");
    static_assert((!TA || (BM >= 64 && BM * ES <= 1024)) && (!TB || (BN >= 64 && BN * ES <= 1024)),
                  "a K-major tile row is 64..1024 bytes");
    static constexpr int KE = BKB / ES; // k rows of a K tile

    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;

    // K-major tiles: k row r of a tile of BX columns sits at r * BX * ES, and its 16-element segments
    // are XOR-ed with bits of r so that the rows touched by one transposing read (fp16: r = 8q + e,
    // e < 4; int8: r = 16q + e, e < 8; the 32 lanes q = 0,1 or q = 2,3 share a pass) fall on distinct banks.
    template <int BX>
    __device__ static __forceinline__ uint32_t tswz(uint32_t r)
    {
        constexpr int P  = BX * ES;
        constexpr int LB = P >= 256 ? 0 : (P == 128 ? 1 : 2); // row bits the pitch already spreads
        const uint32_t full = ES == 2 ? ((r & 3u) | (((r >> 3) & 1u) << 2)) : ((r & 7u) | (((r >> 4) & 1u) << 3));
        return full >> LB;
    }
    // slot j of a thread in a K-major tile: k row and first column of its 16-byte chunk
    template <int BX>
    __device__ static __forceinline__ void tslot(int j, int wave, int lane, uint32_t& r, uint32_t& x)
    {
        constexpr int CPRT = BX * ES / 16, RPW = 64 / CPRT;
        r                  = (uint32_t)((j * NW + wave) * RPW + lane / CPRT);
        const uint32_t pc  = (uint32_t)(lane % CPRT);
        const uint32_t seg = (pc / ES) ^ tswz<BX>(r);
        x                  = seg * 16 + (pc % ES) * (16 / ES);
    }

    // K-contiguous tiles: the 16-byte chunk at position c of staged row r holds chunk c ^ (r & 7) of that
    // row, so the 16 rows read by one MFMA fragment load spread over all LDS banks (measured: no bank
    // conflicts, 256 B/clk).

    __device__ static __forceinline__ void run(const GemmArgs& p, uint8_t* smem)
    {
        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm   = wave / WN;
        const int wn   = wave % WN;

        const int ntiles      = p.tiles_m * p.tiles_n;
        const int nbatch      = p.batch > 0 ? p.batch : 1;
        const int ntiles_all  = ntiles * nbatch; // C tiles of all batches: id = batch * ntiles + tile
        const int gstride     = (int)gridDim.x;
        const uint32_t kbytes = (uint32_t)p.K * ES;
        const int nk_real     = (int)((kbytes + BKB - 1) / BKB);
        const int nk          = nk_real > 0 ? nk_real : 1; // K == 0: one all-zero K tile, C = epilogue(0)

        const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a, p.a_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b, p.b_bytes);
        if constexpr(USE_LUT)
        {
            // (visible to every wave after the prologue's barrier, long before the first epilogue)
            if(p.epi == EPI_REQUANT_RND && p.ksplit == 1)
                requant_lut_fill(smem + NST * STAGE, p.scale_relu, tid, NT);
        }

        // ---- per-thread load slots -------------------------------------------------
        // slot j of this thread fills LDS row (j*NW + wave)*RPI + lane/CPR, chunk position lane%CPR
        // Every slot of a thread sits at the same chunk position: the slot rows differ by
        // multiples of 8 and the swizzle is row & 7, i.e. lane/8 for all of them.
        static_assert(RPI == 8, "one chunk position per thread");
        uint32_t a_off[NLA];  // dense: byte offset of (row, chunk) at K tile 0, or kOutOfRange
        uint32_t a_hw0[NLA]; // im2col: top-left input coordinate of the row's window, (hi0 << 16) | (wi0 & 0xffff)
        int a_d0[IM2COL == 2 ? NLA : 1]; // three spatial dimensions: front input depth of the row's window
        uint32_t b_off[NLB];
        const uint32_t kb = ((uint32_t)(lane % CPR) ^ (uint32_t)((lane / CPR) & 7)) << 4; // chunk byte offset in a K tile
        // K-major operands: k row (within a K tile) of this thread's slot 0; slot j is j * NW * rows-per-load further
        const uint32_t trow_a = TA ? (uint32_t)(wave * (1024 / (BM * ES)) + lane / (BM * ES / 16)) : 0u;
        const uint32_t trow_b = TB ? (uint32_t)(wave * (1024 / (BN * ES)) + lane / (BN * ES / 16)) : 0u;

        // row / column offsets of the tile the LOAD cursor is on (tile >= ntiles: nothing valid)
        auto setup_tile = [&](int tile_id) {
            int tm = 0, tn = 0;
            const bool live = tile_id < ntiles_all;
            int g           = 0;
            if(live)
                tile_of_block(tile_id, p.tiles_m, p.tiles_n, nbatch, g, tm, tn);
            const uint32_t a_batch = (uint32_t)((long)g * p.bsa * ES), b_batch = (uint32_t)((long)g * p.bsb * ES);
#pragma unroll
            for(int j = 0; j < NLA; ++j)
            {
                if constexpr(TA)
                {
                    uint32_t r, x;
                    tslot<BM>(j, wave, lane, r, x);
                    const uint32_t gx = (uint32_t)tm * BM + x;
                    a_off[j] = (live && gx < (uint32_t)p.M) ? a_batch + (r * (uint32_t)p.lda + gx) * ES : kOutOfRange;
                    a_hw0[j] = 0;
                    continue;
                }
                const uint32_t r  = (uint32_t)((j * NW + wave) * RPI + lane / CPR);
                const uint32_t gm = (uint32_t)tm * BM + r;
                const bool ok     = live && gm < (uint32_t)p.M;
                if constexpr(IM2COL == 0)
                {
                    a_off[j] = ok ? a_batch + gm * (uint32_t)p.lda * ES + kb : kOutOfRange;
                    a_hw0[j] = 0;
                }
                else
                {
                    // (cleared up here, not in the branch for rows past M: there it was the branch's last store, and the
                    // compiler folded it with the other branch's last store, that of a_off[j], into ONE store through a
                    // selected address -- which kept both arrays in scratch memory, with scratch loads and waits for all
                    // loads in every K iteration of the 3-D kernels)
                    if constexpr(IM2COL == 2)
                        a_d0[j] = 0;
                    if(ok)
                    {
                        uint32_t img = 0, rem = gm; // img: 2-D image index n, or n * Di + front depth
                        int d0 = 0;
                        if constexpr(IM2COL == 2)
                        {
                            const uint32_t n  = magic_div(gm, p.cv.div_dhowo);
                            const uint32_t r3 = gm - n * p.cv.div_dhowo.d;
                            const uint32_t od = magic_div(r3, p.cv.div_howo);
                            rem               = r3 - od * p.cv.div_howo.d;
                            d0                = (int)od * p.cv.sD - p.cv.pF;
                            img               = (uint32_t)((int)(n * (uint32_t)p.cv.Di) + d0);
                            a_d0[j]           = d0;
                        }
                        else
                        {
                            img = magic_div(gm, p.cv.div_howo);
                            rem = gm - img * p.cv.div_howo.d;
                        }
                        const uint32_t ho  = magic_div(rem, p.cv.div_wo);
                        const uint32_t wo  = rem - ho * p.cv.div_wo.d;
                        const int hi0      = (int)ho * p.cv.sH - p.cv.pT;
                        const int wi0      = (int)wo * p.cv.sW - p.cv.pL;
                        a_hw0[j]           = ((uint32_t)hi0 << 16) | ((uint32_t)wi0 & 0xffffu);
                        // byte offset of the window's top-left (front) pixel; may be "negative" (wraps), the
                        // sum with a valid tap's offset is always inside the tensor
                        a_off[j] = (uint32_t)(((int)(img * (uint32_t)p.cv.Hi) + hi0) * p.cv.Wi + wi0) *
                                   (uint32_t)(p.cv.C * ES);
                    }
                    else
                    {
                        a_hw0[j] = 0xC000C000u; // (-16384, -16384): every tap out of range
                        a_off[j] = 0;
                    }
                }
            }
#pragma unroll
            for(int j = 0; j < NLB; ++j)
            {
                if constexpr(TB)
                {
                    uint32_t r, x;
                    tslot<BN>(j, wave, lane, r, x);
                    const uint32_t gx = (uint32_t)tn * BN + x;
                    b_off[j] = (live && gx < (uint32_t)p.N) ? b_batch + (r * (uint32_t)p.ldb + gx) * ES : kOutOfRange;
                    continue;
                }
                const uint32_t r  = (uint32_t)((j * NW + wave) * RPI + lane / CPR);
                const uint32_t gn = (uint32_t)tn * BN + b_row_to_col(r);
                b_off[j] = (live && gn < (uint32_t)p.N) ? b_batch + gn * (uint32_t)p.ldb * ES + kb : kOutOfRange;
            }
        };

        // Direct global->LDS loads of K tile kt of the load cursor's tile into `stage`, one slot at
        // a time so that the caller can place them between MFMAs. Chunks past K (and whole tiles
        // past the end of the work list) use an out-of-range offset: the hardware writes zeros,
        // and the number of loads in flight stays constant.
        struct LoadCtx
        {
            uint8_t* sa;
            uint8_t* sb;
            uint32_t k0;      // byte offset of the K tile
            uint32_t k0a, k0b; // K-major operands: byte offset of the K tile's first k row
            int klim;          // K-major operands: k rows of this K tile that exist
            uint32_t k_oob;   // top bit set for chunks past K: OR-ed into the offset (arithmetic on
                              // purpose: a select feeding the loads becomes divergent branches)
            int tap_dh, tap_dw; // im2col: decoded ONCE per thread and K tile, every slot of a thread
            int tap_dd;         // sits at the same chunk position
            uint32_t tap_off;
            bool tap_ok;
        };
        auto load_ctx = [&](int kt, int stage) {
            LoadCtx c;
            c.sa    = smem + stage * STAGE;
            c.sb    = c.sa + A_TILE;
            c.k0    = (uint32_t)kt * BKB;
            c.k_oob = (c.k0 + kb < kbytes) ? 0u : kOutOfRange;
            c.k0a   = TA ? (uint32_t)kt * KE * (uint32_t)p.lda * ES : 0u;
            c.k0b   = TB ? (uint32_t)kt * KE * (uint32_t)p.ldb * ES : 0u;
            c.klim  = p.K - kt * KE;
            c.tap_dh = c.tap_dw = c.tap_dd = 0;
            c.tap_off                      = 0;
            c.tap_ok            = true;
            if constexpr(IM2COL != 0)
            {
                const uint32_t ke  = (c.k0 + kb) / ES; // element index along GEMM-K
                uint32_t kyx = ke;
                if constexpr(IM2COL == 2)
                {
                    const uint32_t z = magic_div(ke, p.cv.div_yxc);
                    kyx              = ke - z * p.cv.div_yxc.d;
                    c.tap_dd         = (int)z * p.cv.dD;
                }
                const uint32_t y   = magic_div(kyx, p.cv.div_xc);
                const uint32_t rem = kyx - y * p.cv.div_xc.d;
                const uint32_t x   = magic_div(rem, p.cv.div_c);
                const uint32_t cc  = rem - x * p.cv.div_c.d;
                c.tap_dh           = (int)y * p.cv.dH;
                c.tap_dw           = (int)x * p.cv.dW;
                c.tap_off          = ((uint32_t)((c.tap_dd * p.cv.Hi + c.tap_dh) * p.cv.Wi + c.tap_dw) * (uint32_t)p.cv.C + cc) * ES;
                c.tap_ok           = ke < (uint32_t)p.K;
            }
            return c;
        };
        auto issue_slot = [&](const LoadCtx& c, int slot) { // slot < NLA: A rows, else B rows
            if(slot < NLA)
            {
                const int j = slot;
                uint32_t voff;
                if constexpr(TA)
                    voff = (a_off[j] + c.k0a) | (~(uint32_t)((int)(trow_a + j * NW * (1024 / (BM * ES))) - c.klim) & kOutOfRange);
                else if constexpr(IM2COL == 0)
                    voff = a_off[j] | c.k_oob; // (the K tile's offset travels in the scalar offset: one VALU instruction less)
                else
                {
                    const int hi0 = (int)a_hw0[j] >> 16, wi0 = (int)(a_hw0[j] << 16) >> 16;
                    bool ok = c.tap_ok && (uint32_t)(hi0 + c.tap_dh) < (uint32_t)p.cv.Hi &&
                              (uint32_t)(wi0 + c.tap_dw) < (uint32_t)p.cv.Wi;
                    if constexpr(IM2COL == 2)
                        ok = ok && (uint32_t)(a_d0[j] + c.tap_dd) < (uint32_t)p.cv.Di;
                    voff = (a_off[j] + c.tap_off) | (ok ? 0u : kOutOfRange);
                }
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(c.sa + (j * NW + wave) * 1024), 16,
                                                         voff, (!TA && IM2COL == 0) ? (int)c.k0 : 0, 0, 0);
            }
            else
            {
                const int j         = slot - NLA;
                const uint32_t voff =
                    TB ? (b_off[j] + c.k0b) | (~(uint32_t)((int)(trow_b + j * NW * (1024 / (BN * ES))) - c.klim) & kOutOfRange)
                       : b_off[j] | c.k_oob;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_ptr_t)(c.sb + (j * NW + wave) * 1024), 16,
                                                         voff, TB ? 0 : (int)c.k0, 0, 0);
            }
        };
        auto issue_loads = [&](int kt, int stage) {
            const LoadCtx c = load_ctx(kt, stage);
#pragma unroll
            for(int sl = 0; sl < LPT; ++sl)
                issue_slot(c, sl);
        };

        // A work unit is (K run s, C tile id): unit = s * ntiles_all + id, K tiles [s*nk_per, ...).
        const int nunits = ntiles_all * p.ksplit;
        auto unit_k_range = [&](int unit, int& k_begin, int& k_end) {
            const int sp = unit / ntiles_all;
            k_begin      = sp * p.nk_per;
            k_end        = k_begin + p.nk_per < nk ? k_begin + p.nk_per : nk;
        };
        // load cursor: (unit, kt) of the next K tile to request
        int ld_unit = (int)blockIdx.x, ld_kt = 0, ld_end = nk;
        unit_k_range(ld_unit, ld_kt, ld_end);
        setup_tile(ld_unit < nunits ? ld_unit % ntiles_all : ntiles_all);
        // (kept apart from the issue itself: the branch would split the basic block in which the
        // loads are interleaved with MFMAs)
        auto advance_load_cursor = [&]() {
            if(++ld_kt >= ld_end)
            {
                ld_unit += gstride;
                unit_k_range(ld_unit, ld_kt, ld_end);
                setup_tile(ld_unit < nunits ? ld_unit % ntiles_all : ntiles_all);
            }
        };

        // ---- accumulators ------------------------------------------------------------
        acc_t acc[MT][NG * 4];
#pragma unroll
        for(int i = 0; i < MT; ++i)
#pragma unroll
            for(int t = 0; t < NG * 4; ++t)
                acc[i][t] = acc_t{0, 0, 0, 0};

        // fragment addresses: row = base + lane%16, chunk = 4*ks + lane/16
        const uint32_t frow = (uint32_t)(lane & 15);
        const uint32_t fq   = (uint32_t)(lane >> 4);

        // Fragment r of a k-step, in the order in which the MFMAs of that k-step need them: the B
        // fragments and the first A fragment feed the first MFMA group, the last A fragment only
        // the last one, so the LDS latency of the late reads hides under the early groups.
        // Per-lane parts of the fragment addresses (LDS byte addresses relative to a stage), fixed for the
        // whole kernel; the fragment index and the k-step only add an immediate offset (and, in a K-major
        // tile, flip segment bits: the swizzle is an XOR).
        //   K-contiguous tile: row = wave rows + 16 * fragment + lane % 16, chunk = 4 * ks + lane / 16
        //   K-major tile:      k row = 32 * ks + 8 * (lane / 16) + 4 * h + (lane % 16) / 4   (fp16; h = 0,1)
        //                              64 * ks + 16 * (lane / 16) + 8 * h + (lane % 16) / 2  (int8)
        constexpr int SEGSH = ES == 2 ? 5 : 4;                       // log2 bytes of a 16-element segment
        constexpr int TKS = ES == 2 ? 32 : 64, THALF = ES == 2 ? 4 : 8; // k rows per k-step / per transposing read
        const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
        auto kcontig_part = [&](int wave_row0, int ks) {
            return (uint32_t)(wave_row0 + (int)frow) * BKB + ((((uint32_t)ks * 4 + fq) ^ (frow & 7u)) << 4);
        };
        auto kmajor_part = [&](auto bx, int wave_col0) {
            constexpr int BX = decltype(bx)::value, P = BX * ES;
            const uint32_t e = ES == 2 ? frow >> 2 : frow >> 1, j = ES == 2 ? (frow & 3u) : (frow & 1u);
            const uint32_t r = (ES == 2 ? 8u : 16u) * fq + e;
            return r * P + ((((uint32_t)wave_col0 >> 4) ^ tswz<BX>(r)) << SEGSH) + (j << 3);
        };
        const uint32_t fa0 = TA ? kmajor_part(std::integral_constant<int, BM>{}, wm * WTM) : kcontig_part(wm * WTM, 0);
        const uint32_t fa1 = TA ? fa0 : kcontig_part(wm * WTM, 1);
        const uint32_t fb0 = TB ? kmajor_part(std::integral_constant<int, BN>{}, wn * WTN) : kcontig_part(wn * WTN, 0);
        const uint32_t fb1 = TB ? fb0 : kcontig_part(wn * WTN, 1);
        static_assert((MT & (MT - 1)) == 0 && ((NG * 4) & (NG * 4 - 1)) == 0, "fragment index is XOR-ed into the address");

        // Fragment R of k-step KS, in the order in which the MFMAs of that k-step need them: the B
        // fragments and the first A fragment feed the first MFMA group, the last A fragment only
        // the last one, so the LDS latency of the late reads hides under the early groups.
        // stage_lds: LDS address of the stage.
        auto read_one = [&](uint32_t stage_lds, auto ks_c, auto r_c, i32x4(&af)[MT], i32x4(&bf)[NG * 4]) {
            constexpr int KS = decltype(ks_c)::value, R = decltype(r_c)::value;
            if constexpr(R < NG * 4)
            {
                const uint32_t base = stage_lds + (KS ? fb1 : fb0);
                if constexpr(TB)
                {
                    const uint32_t a = base ^ ((uint32_t)R << SEGSH);
                    const i32x2 lo   = lds_read_tr_b64<ES, A_TILE + KS * TKS * BN * ES>(a);
                    const i32x2 hi   = lds_read_tr_b64<ES, A_TILE + (KS * TKS + THALF) * BN * ES>(a);
                    bf[R]            = i32x4{lo[0], lo[1], hi[0], hi[1]};
                }
                else
                    bf[R] = lds_read_b128<A_TILE + R * 16 * BKB>(base);
            }
            else
            {
                constexpr int I     = R - NG * 4;
                const uint32_t base = stage_lds + (KS ? fa1 : fa0);
                if constexpr(TA)
                {
                    const uint32_t a = base ^ ((uint32_t)I << SEGSH);
                    const i32x2 lo   = lds_read_tr_b64<ES, KS * TKS * BM * ES>(a);
                    const i32x2 hi   = lds_read_tr_b64<ES, (KS * TKS + THALF) * BM * ES>(a);
                    af[I]            = i32x4{lo[0], lo[1], hi[0], hi[1]};
                }
                else
                    af[I] = lds_read_b128<I * 16 * BKB>(base);
            }
        };
        // the kernel's own wait for its fragment reads; nothing may be scheduled across it
        auto wait_frags = [&]() {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mfma_one = [&](int m, const i32x4(&af)[MT], const i32x4(&bf)[NG * 4]) {
            // (B fragments in snake order: one operand stays put across every pair of consecutive MFMAs, which costs
            // measurably less energy on toggling operands than changing both)
            const int i = m / (NG * 4), t = (i & 1) ? NG * 4 - 1 - m % (NG * 4) : m % (NG * 4);
            if constexpr(DT == DT_I8)
                acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[t], af[i], acc[i][t], 0, 0, 0);
            else if constexpr(DT == DT_BF16)
                acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, bf[t]),
                                                                 __builtin_bit_cast(bf16x8, af[i]), acc[i][t], 0, 0, 0);
            else if constexpr(TIED_MFMA)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[i][t]) : "v"(bf[t]), "v"(af[i]));
            else
                acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bf[t]),
                                                                __builtin_bit_cast(f16x8, af[i]), acc[i][t], 0, 0, 0);
        };
        // With TIED_MFMA: between the K loop's last MFMAs and the epilogue's first look at their results the wait
        // states a matrix result needs before a vector instruction or a store may read it (at most 18; 32 are spent,
        // once per tile), and between the epilogue's zeroing of the accumulators and the next MFMA the few that a
        // vector result needs before a matrix instruction reads it as its addend. Every accumulator passes through an
        // empty statement of its own behind the idle cycles, which is what keeps the two sides apart.
        auto acc_handover = [&](auto to_epilogue) {
            if constexpr(TIED_MFMA)
            {
                if constexpr(decltype(to_epilogue)::value)
                    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
                for(int i = 0; i < MT; ++i)
#pragma unroll
                    for(int t = 0; t < NG * 4; ++t)
                        asm volatile("" : "+v"(acc[i][t]));
                if constexpr(!decltype(to_epilogue)::value)
                    asm volatile("s_nop 7" ::: "memory");
            }
        };

        // One half of a K-tile iteration, written as LPT groups pinned in source order
        // (sched_barrier): group g = [one direct global->LDS load of the K tile after next]
        // + [its share of the LDS reads of the NEXT k-step] + [its share of the MFMAs of the CURRENT
        // k-step]. The loads must not be issued back to back: a burst of eight 1 KB loads per wave
        // fills the texture-address FIFOs (SQ_VMEM_TA_ADDR/CMD_FIFO_FULL), the in-order wave blocks
        // on VMEM issue, and its MFMAs wait behind it.
        auto half_step = [&](auto with_loads, const LoadCtx& lc, const i32x4(&caf)[MT], const i32x4(&cbf)[NG * 4],
                             uint32_t nstage_lds, auto nks, i32x4(&naf)[MT], i32x4(&nbf)[NG * 4]) {
            // The reads are over two groups before the end of the half; the first half of an iteration
            // starts its reads one group late.
            constexpr int NGRP = LPT, NR = MT + NG * 4, NM = MT * NG * 4;
            constexpr int RG  = NGRP >= 4 ? NGRP - 2 : NGRP;
            constexpr int RG0 = (NGRP >= 4 && !decltype(with_loads)::value) ? 1 : 0;
            static_for<NGRP>([&](auto g_c) {
                constexpr int g = decltype(g_c)::value;
                if constexpr(decltype(with_loads)::value)
                    issue_slot(lc, g);
                constexpr int gr = g - RG0 < 0 ? 0 : (g - RG0 > RG ? RG : g - RG0); // read groups done before g
                constexpr int gn = g + 1 - RG0 < 0 ? 0 : (g + 1 - RG0 > RG ? RG : g + 1 - RG0);
                constexpr int r0 = gr * NR / RG, r1 = gn * NR / RG;
                static_for<r1 - r0>([&](auto r_c) {
                    read_one(nstage_lds, nks, std::integral_constant<int, r0 + decltype(r_c)::value>{}, naf, nbf);
                });
#pragma unroll
                for(int m = g * NM / NGRP; m < (g + 1) * NM / NGRP; ++m)
                    mfma_one(m, caf, cbf);
                __builtin_amdgcn_sched_barrier(0);
            });
        };

        // ---- epilogue: registers -> global, 16 consecutive columns per lane -------------
        const bool vec_ok = ((reinterpret_cast<uintptr_t>(p.c) | ((uintptr_t)p.ldc * ES) |
                              (nbatch > 1 ? (uintptr_t)p.bsc * ES : 0)) & 15u) == 0;
        const bool nt     = p.nt_store != 0;
        const bool dvec_ok = ((reinterpret_cast<uintptr_t>(p.d0) | ((uintptr_t)p.ldd0 * ES) |
                               reinterpret_cast<uintptr_t>(p.d1) | ((uintptr_t)p.ldd1 * ES)) & 15u) == 0;
        auto epilogue = [&](int unit) {
            int tm, tn, bi;
            tile_of_block(unit % ntiles_all, p.tiles_m, p.tiles_n, nbatch, bi, tm, tn);
            // (a K split is never combined with a batch: the slices are [run][M][N])
            acc_t* slice = reinterpret_cast<acc_t*>(reinterpret_cast<uint8_t*>(p.ws) +
                                                    (size_t)(unit / ntiles_all) * p.M * p.N * 4);
            uint8_t* c_batch = reinterpret_cast<uint8_t*>(p.c) + (size_t)bi * p.bsc * ES;
            // Per-column requant scales (the FUSED variant of the int8 kernel: compiled into the plain one it cost the
            // im2col instances ten more spilled SGPRs and 7 - 10 % on the conv and LLM shapes): a loop nest of its own,
            // column group outermost, so that the 16 scales of the lane's columns are fetched once per group and before
            // that group's stores (a load issued after a store waits for it) and only 16 registers hold them.
            if constexpr(DT == DT_I8 && FUSED)
            {
                if(epi_per_column_scale(p.epi) && p.ksplit == 1)
                {
                    const __amdgpu_buffer_rsrc_t rs = make_rsrc(p.d0, (uint32_t)p.N * 4u);
                    const bool relu                 = p.epi == EPI_RELU_MUL2_CLAMP;
#pragma unroll
                    for(int g = 0; g < NG; ++g)
                    {
                        const int n0 = tn * BN + wn * WTN + 64 * g + 16 * (lane >> 4);
                        float sc[16];
                        load_col_scales(rs, n0, sc);
                        // (awaited here, where every lane passes: the uses sit under a condition, and a load that the
                        // compiler cannot prove consumed makes it wait for all loads in every K iteration)
                        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
#pragma unroll
                        for(int i = 0; i < MT; ++i)
                        {
                            const int m = tm * BM + wm * WTM + 16 * i + (lane & 15);
                            if(m < p.M && n0 < p.N)
                            {
                                const i32x4 v[4] = {acc[i][g * 4], acc[i][g * 4 + 1], acc[i][g * 4 + 2], acc[i][g * 4 + 3]};
                                store_row16_i8_cols(reinterpret_cast<int8_t*>(c_batch) + (size_t)m * p.ldc, n0, p.N, vec_ok,
                                                    v, sc, relu, nt);
                            }
#pragma unroll
                            for(int t = 0; t < 4; ++t)
                                acc[i][g * 4 + t] = acc_t{0, 0, 0, 0};
                        }
                    }
                    return;
                }
            }
#pragma unroll
            for(int i = 0; i < MT; ++i)
            {
                const int m = tm * BM + wm * WTM + 16 * i + (lane & 15);
#pragma unroll
                for(int g = 0; g < NG; ++g)
                {
                    const int n0 = tn * BN + wn * WTN + 64 * g + 16 * (lane >> 4);
                    if(m < p.M && n0 < p.N)
                    {
                        if(p.ksplit > 1)
                        {
                            // raw accumulators, 16 consecutive columns = 64 bytes per lane
                            uint8_t* wrow = reinterpret_cast<uint8_t*>(slice) + ((size_t)m * p.N + n0) * 4;
                            if(n0 + 16 <= p.N && (p.N & 3) == 0)
                            {
#pragma unroll
                                for(int t = 0; t < 4; ++t)
                                    reinterpret_cast<acc_t*>(wrow)[t] = acc[i][g * 4 + t];
                            }
                            else
                            {
#pragma unroll
                                for(int e = 0; e < 16; ++e)
                                    if(n0 + e < p.N)
                                        reinterpret_cast<decltype(acc[0][0][0] + 0)*>(wrow)[e] = acc[i][g * 4 + e / 4][e % 4];
                            }
                        }
                        else if constexpr(DT == DT_I8)
                        {
                            int8_t* crow = reinterpret_cast<int8_t*>(c_batch) + (size_t)m * p.ldc;
                            const i32x4 v[4] = {acc[i][g * 4], acc[i][g * 4 + 1], acc[i][g * 4 + 2],
                                                acc[i][g * 4 + 3]};
                            if(p.epi == EPI_REQUANT_RND && USE_LUT)
                                store_row16_i8_lut(crow, n0, p.N, vec_ok, v, p.scale_gemm,
                                                   (uint32_t)(uintptr_t)(lds_ptr_t)smem + (uint32_t)(NST * STAGE), nt);
                            else if(p.epi == EPI_REQUANT_RND)
                                store_row16_i8<EPI_REQUANT_RND>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                            else if(p.epi == EPI_REQUANT_CK)
                                store_row16_i8<EPI_REQUANT_CK>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                            else
                                store_row16_i8<EPI_PASSTHROUGH>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                        }
                        else
                        {
                            const f32x4 v[4] = {acc[i][g * 4], acc[i][g * 4 + 1], acc[i][g * 4 + 2],
                                                acc[i][g * 4 + 3]};
                            if constexpr(DT == DT_BF16)
                                store_row16_f16(reinterpret_cast<__bf16*>(c_batch) + (size_t)m * p.ldc, n0, p.N, vec_ok,
                                                v, nt);
                            else
                                store_row16_f16(reinterpret_cast<_Float16*>(c_batch) + (size_t)m * p.ldc, n0, p.N,
                                                vec_ok, v, nt);
                        }
                    }
#pragma unroll
                    for(int t = 0; t < 4; ++t)
                        acc[i][g * 4 + t] = acc_t{0, 0, 0, 0};
                }
            }
        };

        // Epilogue of the fused add / ReLU modes (fp16, no K split). A load issued after a store
        // has to wait for that store as well (one counter, no ordering between the two kinds), so
        // the D values are fetched in chunks of CH accumulator rows BEFORE any store of the chunk:
        // a bias row once for the whole tile, per-row tensors (residual) chunk by chunk.
        // (which tensors are per-row is a compile-time property of each variant: registers are only
        // set aside for what is fetched)
        // (so is the functor family: EXT = false builds the add / ReLU modes alone, EXT = true the scaled and GELU ones)
        // The functor is a compile-time constant of each copy: as a run-time value every output paid for both add / ReLU
        // forms and the selects between them (bias + ReLU on a 200704 x 256 x 64 problem: 43.4 us against 29.3 plain).
        auto epilogue_fused = [&](int unit, auto chunk_rows, auto d0_row_tensor, auto mode_c) {
            constexpr int CH          = decltype(chunk_rows)::value < MT ? decltype(chunk_rows)::value : MT;
            constexpr bool d0_per_row = decltype(d0_row_tensor)::value;
            using functor             = decltype(mode_c);
            constexpr bool has_d1     = functor::has_d1;
            constexpr bool EXT        = functor::ext;
            const int mode            = functor::mode(p);
            int tm, tn, bi; // (the fused epilogues are never combined with a batch)
            tile_of_block(unit % ntiles, p.tiles_m, p.tiles_n, 1, bi, tm, tn);
            const _Float16* d0 = reinterpret_cast<const _Float16*>(p.d0);
            const _Float16* d1 = reinterpret_cast<const _Float16*>(p.d1);
            const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
            auto load16 = [&](const _Float16* row, int n0, f16x8& lo, f16x8& hi) {
                if(dvec_ok && n0 + 16 <= p.N)
                {
                    lo = *reinterpret_cast<const f16x8*>(row + n0);
                    hi = *reinterpret_cast<const f16x8*>(row + n0 + 8);
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < 8; ++e)
                    {
                        lo[e] = n0 + e < p.N ? row[n0 + e] : (_Float16)0;
                        hi[e] = n0 + 8 + e < p.N ? row[n0 + 8 + e] : (_Float16)0;
                    }
                }
            };
            auto col0 = [&](int g) { return tn * BN + wn * WTN + 64 * g + 16 * (lane >> 4); };
            f16x8 b_lo[NG], b_hi[NG];
#pragma unroll
            for(int g = 0; g < NG; ++g)
            {
                b_lo[g] = b_hi[g] = zero8;
                if(!d0_per_row && col0(g) < p.N)
                    load16(d0, col0(g), b_lo[g], b_hi[g]);
            }
            // The D values are awaited where every lane passes, right behind their loads (they are the youngest
            // requests, so the first use would wait for as much). Left to the uses, which sit under the same conditions
            // as the loads but not provably so, the compiler sees a path on which a load is still on its way when the
            // K loop starts over, and guards that loop's fragment registers with a wait for all loads in every iteration.
            auto d_values_landed = [] { __builtin_amdgcn_s_waitcnt(0x0F70); /* vmcnt(0), nothing else */ };
            if constexpr(!d0_per_row)
                d_values_landed();
#pragma unroll
            for(int i0 = 0; i0 < MT; i0 += CH)
            {
                f16x8 x_lo[d0_per_row ? CH : 1][NG], x_hi[d0_per_row ? CH : 1][NG];
                f16x8 y_lo[has_d1 ? CH : 1][NG], y_hi[has_d1 ? CH : 1][NG];
#pragma unroll
                for(int c = 0; c < CH; ++c)
#pragma unroll
                    for(int g = 0; g < NG; ++g)
                    {
                        const int m     = tm * BM + wm * WTM + 16 * (i0 + c) + (lane & 15);
                        const bool live = m < p.M && col0(g) < p.N;
                        if constexpr(d0_per_row)
                        {
                            x_lo[c][g] = x_hi[c][g] = zero8;
                            if(live)
                                load16(d0 + (size_t)m * p.ldd0, col0(g), x_lo[c][g], x_hi[c][g]);
                        }
                        if constexpr(has_d1)
                        {
                            y_lo[c][g] = y_hi[c][g] = zero8;
                            if(live)
                                load16(d1 + (size_t)m * p.ldd1, col0(g), y_lo[c][g], y_hi[c][g]);
                        }
                    }
                if constexpr(d0_per_row || has_d1)
                    d_values_landed();
#pragma unroll
                for(int c = 0; c < CH; ++c)
#pragma unroll
                    for(int g = 0; g < NG; ++g)
                    {
                        const int i = i0 + c;
                        const int m = tm * BM + wm * WTM + 16 * i + (lane & 15);
                        if(m < p.M && col0(g) < p.N)
                        {
                            f32x4 v[4];
#pragma unroll
                            for(int t = 0; t < 4; ++t)
#pragma unroll
                                for(int j = 0; j < 4; ++j)
                                {
                                    const int e   = t * 4 + j;
                                    const int cx  = d0_per_row ? c : 0, cy = has_d1 ? c : 0;
                                    const float x = d0_per_row ? (float)(e < 8 ? x_lo[cx][g][e & 7] : x_hi[cx][g][e & 7])
                                                               : (float)(e < 8 ? b_lo[g][e & 7] : b_hi[g][e & 7]);
                                    const float y = has_d1 ? (float)(e < 8 ? y_lo[cy][g][e & 7] : y_hi[cy][g][e & 7]) : 0.0f;
                                    v[t][j] = epi_f16_value<EXT>(mode, acc[i][g * 4 + t][j], x, y, p.scale_gemm, p.scale_relu);
                                }
                            _Float16* crow = reinterpret_cast<_Float16*>(p.c) + (size_t)m * p.ldc;
                            store_row16_f16(crow, col0(g), p.N, vec_ok, v, nt);
                        }
#pragma unroll
                        for(int t = 0; t < 4; ++t)
                            acc[i][g * 4 + t] = acc_t{0, 0, 0, 0};
                    }
            }
        };

        // K-major B: MFMA tile t of a 64-column group covered columns 16t..16t+15, so the lane in 16-lane
        // row q holds columns 16t + 4q + (0..3). A 4x4 transpose between t and q (two butterfly stages of
        // v_permlane32_swap / v_permlane16_swap) gives lane row q the columns 16q + 4t + (0..3) -- the
        // ownership the epilogues are written for.
        auto transpose_acc = [&]() {
#pragma unroll
            for(int i = 0; i < MT; ++i)
#pragma unroll
                for(int g = 0; g < NG; ++g)
#pragma unroll
                    for(int e = 0; e < 4; ++e)
                    {
                        uint32_t x[4];
#pragma unroll
                        for(int t = 0; t < 4; ++t)
                        {
                            // (through a scalar temporary: a bit cast applied directly to a vector-element
                            // lvalue reads element 0)
                            const auto v = acc[i][g * 4 + t][e];
                            x[t]         = __builtin_bit_cast(uint32_t, v);
                        }
                        // rows 2,3 of x[t] <-> rows 0,1 of x[t + 2]
                        auto s02 = __builtin_amdgcn_permlane32_swap(x[0], x[2], false, false);
                        auto s13 = __builtin_amdgcn_permlane32_swap(x[1], x[3], false, false);
                        // odd rows of the first <-> even rows of the second
                        auto u01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
                        auto u23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
                        x[0] = u01[0], x[1] = u01[1], x[2] = u23[0], x[3] = u23[1];
#pragma unroll
                        for(int t = 0; t < 4; ++t)
                            acc[i][g * 4 + t][e] = __builtin_bit_cast(decltype(acc[0][0][0] + 0), x[t]);
                    }
        };

        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };

        // Register double buffer over the two k-steps of a K tile. The barrier sits between
        // them: by then every wave has pulled ALL of the current K tile into registers, so its
        // stage can be refilled right away, and the first fragments of the next K tile (of this
        // or of the next C tile) are read while the second half is still being multiplied.
        i32x4 af0[MT], bf0[NG * 4], af1[MT], bf1[NG * 4];

#pragma unroll
        for(int st = 0; st < NST; ++st)
        {
            issue_loads(ld_kt, st);
            advance_load_cursor();
        }
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 1) * LPT) : "memory");
        barrier();
        static_for<MT + NG * 4>([&](auto r_c) { read_one(smem_lds, std::integral_constant<int, 0>{}, r_c, af0, bf0); });

        int kt = 0, kt_end = nk;
        int st_cur = 0;       // stage of the K tile being multiplied
        bool drain = false;   // C stores are in flight: the next wait cannot count loads
        unit_k_range((int)blockIdx.x, kt, kt_end);
        for(int unit = (int)blockIdx.x; unit < nunits;)
        {
            const int st_next  = st_cur + 1 == NST ? 0 : st_cur + 1;
            // first fragments of this K tile (read in the previous half-iteration / the prologue)
            wait_frags();
            half_step(std::false_type{}, LoadCtx{}, af0, bf0, smem_lds + (uint32_t)(st_cur * STAGE),
                      std::integral_constant<int, 1>{}, af1, bf1);

            // The direct loads of a wave retire in order: once at most NST-2 K tiles' worth are in
            // flight, the next K tile has landed. C stores of an epilogue share the counter and are
            // not ordered against loads, so the first wait after an epilogue drains everything.
            // The current K tile is entirely in registers by now (lgkmcnt).
            if(drain)
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            else
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NST - 2) * LPT) : "memory");
            __builtin_amdgcn_sched_barrier(0);
            drain = false;
            barrier();

            const LoadCtx lc = load_ctx(ld_kt, st_cur);
            half_step(std::true_type{}, lc, af1, bf1, smem_lds + (uint32_t)(st_next * STAGE),
                      std::integral_constant<int, 0>{}, af0, bf0);
            advance_load_cursor();

            st_cur = st_next;
            if(++kt >= kt_end)
            {
                acc_handover(std::true_type{});
                if constexpr(TB)
                    transpose_acc();
                if constexpr(FUSED && DT == DT_F16)
                {
                    if(p.epi == EPI_PASSTHROUGH || p.ksplit > 1)
                        epilogue(unit);
                    else
                    {
                        using std::integral_constant;
                        using std::false_type;
                        using std::true_type;
                        const bool d0_rows = p.ldd0 != 0;
                        // chunks of fragment rows whose D values are fetched together: all of them for a bias row alone,
                        // two with one per-row tensor, one with two
                        auto with_functor = [&](auto mode_c) {
                            constexpr bool resi = decltype(mode_c)::has_d1;
                            if(!d0_rows)
                                epilogue_fused(unit, integral_constant<int, (resi ? 2 : MT)>{}, false_type{}, mode_c);
                            else
                                epilogue_fused(unit, integral_constant<int, (resi ? 1 : 2)>{}, true_type{}, mode_c);
                        };
                        if constexpr(BM * BN >= 256 * 256)
                        {
                            // (the instance that holds 128 accumulators per lane fills the register file already: with
                            // a copy of the epilogue per functor it spills)
                            auto by_operands = [&](auto extended) {
                                constexpr bool EXT = decltype(extended)::value;
                                if(epi_has_d1(p.epi))
                                    with_functor(FunctorOf<true, EXT, IM2COL != 0>{});
                                else if(!EXT && IM2COL == 0 && p.epi == EPI_ADD_RELU)
                                    with_functor(FunctorOf<false, false, true>{});
                                else
                                    with_functor(FunctorOf<false, EXT, IM2COL != 0>{});
                            };
                            if(IM2COL == 0 && p.epi >= EPI_BILINEAR)
                            {
                                if constexpr(IM2COL == 0)
                                    by_operands(true_type{});
                            }
                            else
                                by_operands(false_type{});
                        }
                        else if(p.epi == EPI_ADD_RELU)
                            with_functor(FunctorIs<EPI_ADD_RELU>{});
                        else if(p.epi == EPI_ADD_RELU_ADD)
                            with_functor(FunctorIs<EPI_ADD_RELU_ADD>{});
                        else
                        {
                            // (the conv operators take the two functors above only)
                            if constexpr(IM2COL == 0)
                            {
                                if(p.epi == EPI_CSHUFFLE_ADD_RELU)
                                    with_functor(FunctorIs<EPI_CSHUFFLE_ADD_RELU>{});
                                else if(p.epi == EPI_BILINEAR)
                                    with_functor(FunctorIs<EPI_BILINEAR>{});
                                else
                                    with_functor(FunctorIs<EPI_ADD_ADD_FASTGELU>{});
                            }
                        }
                    }
                }
                else
                    epilogue(unit);
                acc_handover(std::false_type{});
                drain = true;
                unit += gstride;
                unit_k_range(unit, kt, kt_end);
            }
        }
        // the trailing (all-zero) loads still target LDS: let them retire before the workgroup
        // gives its LDS back
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
};

// Second pass of a split-K launch: C = epilogue(sum over the K runs of the workspace slices).
// One thread per 16 consecutive columns of a row, slices added in run order (deterministic).
template <int DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs p)
{
    using acc_t   = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    constexpr int ES = DT == DT_I8 ? 1 : 2;
    const int groups_per_row = (p.N + 15) / 16;
    const long gid = (long)blockIdx.x * 256 + threadIdx.x;
    if(gid >= (long)p.M * groups_per_row)
        return;
    const int m  = (int)(gid / groups_per_row);
    const int n0 = (int)(gid - (long)m * groups_per_row) * 16;
    acc_t v[4];
#pragma unroll
    for(int t = 0; t < 4; ++t)
        v[t] = acc_t{0, 0, 0, 0};
    const bool full = n0 + 16 <= p.N && (p.N & 3) == 0;
    for(int sp = 0; sp < p.ksplit; ++sp)
    {
        const uint8_t* wrow = reinterpret_cast<const uint8_t*>(p.ws) + (((size_t)sp * p.M + m) * p.N + n0) * 4;
        if(full)
        {
#pragma unroll
            for(int t = 0; t < 4; ++t)
            {
                const acc_t w = reinterpret_cast<const acc_t*>(wrow)[t];
                v[t][0] += w[0], v[t][1] += w[1], v[t][2] += w[2], v[t][3] += w[3];
            }
        }
        else
        {
#pragma unroll
            for(int e = 0; e < 16; ++e)
                if(n0 + e < p.N)
                    v[e / 4][e % 4] += reinterpret_cast<const decltype(v[0][0] + 0)*>(wrow)[e];
        }
    }
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(p.c) | ((uintptr_t)p.ldc * ES)) & 15u) == 0;
    if constexpr(DT == DT_I8)
    {
        int8_t* crow = reinterpret_cast<int8_t*>(p.c) + (size_t)m * p.ldc;
        if(epi_per_column_scale(p.epi))
        {
            float sc[16];
            load_col_scales(make_rsrc(p.d0, (uint32_t)p.N * 4u), n0, sc);
            store_row16_i8_cols(crow, n0, p.N, vec_ok, v, sc, p.epi == EPI_RELU_MUL2_CLAMP);
        }
        else if(p.epi == EPI_REQUANT_RND)
            store_row16_i8<EPI_REQUANT_RND>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu);
        else if(p.epi == EPI_REQUANT_CK)
            store_row16_i8<EPI_REQUANT_CK>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu);
        else
            store_row16_i8<EPI_PASSTHROUGH>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu);
    }
    else if constexpr(DT == DT_BF16)
        store_row16_f16(reinterpret_cast<__bf16*>(p.c) + (size_t)m * p.ldc, n0, p.N, vec_ok, v);
    else
    {
        _Float16* crow = reinterpret_cast<_Float16*>(p.c) + (size_t)m * p.ldc;
        if(p.epi == EPI_PASSTHROUGH)
            store_row16_f16(crow, n0, p.N, vec_ok, v);
        else
        {
            const bool dvec_ok = ((reinterpret_cast<uintptr_t>(p.d0) | ((uintptr_t)p.ldd0 * ES) |
                                   reinterpret_cast<uintptr_t>(p.d1) | ((uintptr_t)p.ldd1 * ES)) & 15u) == 0;
            store_row16_f16_fused(crow, n0, p.N, vec_ok, v, p.epi,
                                  reinterpret_cast<const _Float16*>(p.d0) + (size_t)m * p.ldd0,
                                  p.d1 ? reinterpret_cast<const _Float16*>(p.d1) + (size_t)m * p.ldd1 : nullptr,
                                  dvec_ok, false, p.scale_gemm, p.scale_relu);
        }
    }
}

template <int DT, int BM, int BN, int WM, int WN, int BKB, int NST, int IM2COL, bool TA = false, bool TB = false,
          bool FUSED = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_tile_kernel(const GemmArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_smem[];
    GemmTile<DT, BM, BN, WM, WN, BKB, NST, IM2COL, TA, TB, FUSED>::run(p, ckx_smem);
}

} // namespace ckx
