// Conv2d forward for the first layer of an image network: C = 3 input channels, 7 x 7 filter, stride 2, padding 3,
// K = 64 output channels, NHWC / KYXC / NHWK (ResNet-50's stem: the first line of the reference's
// script/profile_resnet50.sh; device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:224-301 reaches it through its OddC
// specialisation with one-element loads). A pixel is 6 (fp16) or 3 (int8) bytes: no 16-byte vector of the input is
// aligned to a filter tap, and the implicit-GEMM tile kernels cannot load it. Here
//   * a workgroup (four waves) walks bands of TH output rows of an image; the band's 2 TH + 5 input rows are copied
//     into LDS once, each pixel PADDED TO FOUR CHANNELS (8 / 4 bytes) with the zero padding of the borders written out,
//     so that the window row of output pixel wo starts at byte 16 wo (fp16) / 8 wo (int8) of the LDS row: aligned reads;
//   * GEMM-K runs over (y, x', c') with x' = 0..7, c' = 0..3 -- 32 elements per filter row, the taps x' = 7 and c' = 3
//     with zero weights: one MFMA k-step per filter row (fp16, 7 k-steps of 32) or per two filter rows (int8, 4 k-steps
//     of 64, the eighth row all zeros); an A fragment is one ds_read_b128 (fp16) / two ds_read_b64 (int8);
//   * the weights stay in registers for the life of the workgroup, as B fragments in that K order and with the output
//     channels permuted so that a lane ends with 16 consecutive channels of one pixel (four lanes = one whole pixel of
//     64 channels: 128 / 64 contiguous bytes per pixel, 2 / 1 KB per MFMA tile);
//   * several workgroups per CU overlap one's copy phase with another's MFMAs and stores.
// Algorithmic traffic is the output (N x 112 x 112 x 64) by far: the layer is bound by HBM writes.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct ConvStemArgs
{
    const void* in;
    const void* wei;
    void* out;
    const void* bias; // fp16 [64] (EPI_ADD_RELU)
    int N, Hi, Wi, Ho, Wo;
    int epi;          // fp16: EPI_PASSTHROUGH, EPI_ADD_RELU; int8: EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND
    float scale_gemm, scale_relu;
    int nt_store;
};

template <int DT>
struct ConvStem
{
    static_assert(DT == DT_F16 || DT == DT_I8, "fp16 or int8");
    static constexpr int ES = DT == DT_I8 ? 1 : 2;
    static constexpr int C = 3, Y = 7, X = 7, S = 2, PAD = 3, KOUT = 64;
    static constexpr int TH = 4, ROWS = S * TH + Y - S; // input rows of a band
    static constexpr int PX = 4 * ES;                   // bytes of a padded pixel in LDS
    static constexpr int NKS = DT == DT_I8 ? 4 : 7;     // MFMA k-steps per output tile
    static constexpr int NTHR = 256, NW = 4;
    using acc_t  = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    using elem_t = typename std::conditional<DT == DT_I8, int8_t, _Float16>::type;

    // bytes of an LDS row: windows of 8 padded pixels for every output pixel of the (padded) tile row
    __host__ __device__ static int slot_bytes(int Wo) { return ((Wo + 15) / 16 * 16) * S * PX + 8 * PX; }
    __host__ __device__ static int lds_bytes(int Wo) { return ROWS * slot_bytes(Wo); }

    __device__ static __forceinline__ void run(const ConvStemArgs& p, uint8_t* smem)
    {
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t r = lane & 15, q = lane >> 4;
        const int slot    = slot_bytes(p.Wo);
        const int wtiles  = (p.Wo + 15) / 16;
        const int bands   = (p.Ho + TH - 1) / TH;
        const int nunits  = p.N * bands;
        const elem_t* in  = reinterpret_cast<const elem_t*>(p.in);
        const elem_t* wei = reinterpret_cast<const elem_t*>(p.wei);

        // ---- the weights as B fragments: N tile t, k-step ks; lane (r, q) holds the 8 (16) K elements 8 q .. (16 q ..)
        // of LDS-order row 16 t + r, which is output channel b_row_to_col(16 t + r)
        i32x4 bfr[4][NKS];
#pragma unroll
        for(int t = 0; t < 4; ++t)
        {
            const int n = (int)b_row_to_col((uint32_t)(16 * t) + r);
#pragma unroll
            for(int ks = 0; ks < NKS; ++ks)
            {
                if constexpr(DT == DT_F16)
                {
                    f16x8 v;
#pragma unroll
                    for(int e = 0; e < 8; ++e)
                    {
                        const int j = 8 * (int)q + e, x = j >> 2, c = j & 3; // k' = 32 ks + j: filter row ks
                        v[e]        = (x < X && c < C) ? wei[((n * Y + ks) * X + x) * C + c] : (_Float16)0;
                    }
                    bfr[t][ks] = __builtin_bit_cast(i32x4, v);
                }
                else
                {
                    typedef int8_t i8x16 __attribute__((ext_vector_type(16)));
                    i8x16 v;
                    const int y = 2 * ks + ((int)q >> 1); // k' = 64 ks + 16 q + e: filter rows 2 ks, 2 ks + 1
#pragma unroll
                    for(int e = 0; e < 16; ++e)
                    {
                        const int j = 16 * ((int)q & 1) + e, x = j >> 2, c = j & 3;
                        v[e]        = (y < Y && x < X && c < C) ? wei[((n * Y + y) * X + x) * C + c] : (int8_t)0;
                    }
                    bfr[t][ks] = __builtin_bit_cast(i32x4, v);
                }
            }
        }
        f32x4 bias[4];
#pragma unroll
        for(int t = 0; t < 4; ++t)
#pragma unroll
            for(int j = 0; j < 4; ++j)
                bias[t][j] = (DT == DT_F16 && p.epi == EPI_ADD_RELU) ? (float)reinterpret_cast<const _Float16*>(p.bias)[16 * q + 4 * t + j] : 0.0f;

        const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
        const bool nt           = p.nt_store != 0;
        const bool vec_ok       = (reinterpret_cast<uintptr_t>(p.out) & 15u) == 0;

        for(int unit = (int)blockIdx.x; unit < nunits; unit += (int)gridDim.x)
        {
            const int n = unit / bands, ho0 = (unit - n * bands) * TH;
            const int hi0 = ho0 * S - PAD;
            // ---- copy the band: padded pixel slot pp of LDS row rr <- input pixel (hi0 + rr, pp - PAD), zeros outside
            const int npx = slot / PX;
            __syncthreads(); // (every wave is done with the previous band)
            for(int i = tid; i < ROWS * npx; i += NTHR)
            {
                const int rr = i / npx, pp = i - rr * npx;
                const int hi = hi0 + rr, wi = pp - PAD;
                const bool ok = hi >= 0 && hi < p.Hi && wi >= 0 && wi < p.Wi;
                const elem_t* src = in + ((size_t)(n * p.Hi + (ok ? hi : 0)) * p.Wi + (ok ? wi : 0)) * C;
                if constexpr(DT == DT_F16)
                {
                    typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
                    f16x4 v = {0, 0, 0, 0};
                    if(ok)
                        v[0] = src[0], v[1] = src[1], v[2] = src[2];
                    *reinterpret_cast<f16x4*>(smem + rr * slot + pp * PX) = v;
                }
                else
                {
                    typedef int8_t i8x4 __attribute__((ext_vector_type(4)));
                    i8x4 v = {0, 0, 0, 0};
                    if(ok)
                        v[0] = src[0], v[1] = src[1], v[2] = src[2];
                    *reinterpret_cast<i8x4*>(smem + rr * slot + pp * PX) = v;
                }
            }
            __syncthreads();
            // ---- output tiles of the band: 16 consecutive pixels of one output row each, dealt to the waves
            for(int tile = wave; tile < TH * wtiles; tile += NW)
            {
                const int hl = tile / wtiles, wt = tile - hl * wtiles;
                const int ho = ho0 + hl;
                if(ho >= p.Ho)
                    continue;
                // window of pixel wo = 16 wt + r: LDS row 2 hl + y, bytes [S PX wo, S PX wo + 8 PX)
                const uint32_t base = smem_lds + (uint32_t)(S * hl * slot) + (uint32_t)(S * PX) * (16u * wt + r);
                i32x4 af[NKS];
#pragma unroll
                for(int ks = 0; ks < NKS; ++ks)
                {
                    if constexpr(DT == DT_F16)
                        af[ks] = *reinterpret_cast<const i32x4*>(smem + (base - smem_lds) + ks * slot + 16 * q);
                    else
                    {
                        const int y = 2 * ks + ((int)q >> 1) < Y ? 2 * ks + ((int)q >> 1) : Y - 1; // (row 7: zero weights)
                        const i32x2* s2 = reinterpret_cast<const i32x2*>(smem + (base - smem_lds) + y * slot + 16 * (q & 1));
                        const i32x2 lo = s2[0], hi = s2[1];
                        af[ks]         = i32x4{lo[0], lo[1], hi[0], hi[1]};
                    }
                }
                acc_t acc[4];
#pragma unroll
                for(int t = 0; t < 4; ++t)
                    acc[t] = acc_t{0, 0, 0, 0};
#pragma unroll
                for(int ks = 0; ks < NKS; ++ks)
#pragma unroll
                    for(int t = 0; t < 4; ++t)
                    {
                        if constexpr(DT == DT_I8)
                            acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bfr[t][ks], af[ks], acc[t], 0, 0, 0);
                        else
                            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bfr[t][ks]),
                                                                            __builtin_bit_cast(f16x8, af[ks]), acc[t], 0, 0, 0);
                    }
                // ---- lane (pixel r of the tile, q): channels 16 q .. 16 q + 15
                const int wo = 16 * wt + (int)r;
                if(wo >= p.Wo)
                    continue;
                elem_t* crow = reinterpret_cast<elem_t*>(p.out) + ((size_t)(n * p.Ho + ho) * p.Wo + wo) * KOUT;
                if constexpr(DT == DT_F16)
                {
                    if(p.epi == EPI_ADD_RELU)
                    {
#pragma unroll
                        for(int t = 0; t < 4; ++t)
#pragma unroll
                            for(int j = 0; j < 4; ++j)
                                acc[t][j] = __builtin_fmaxf(acc[t][j] + bias[t][j], 0.0f);
                    }
                    store_row16_f16(crow, 16 * (int)q, KOUT, vec_ok, acc, nt);
                }
                else
                {
                    if(p.epi == EPI_REQUANT_RND)
                        store_row16_i8<EPI_REQUANT_RND>(crow, 16 * (int)q, KOUT, vec_ok, acc, p.scale_gemm, p.scale_relu, nt);
                    else if(p.epi == EPI_REQUANT_CK)
                        store_row16_i8<EPI_REQUANT_CK>(crow, 16 * (int)q, KOUT, vec_ok, acc, p.scale_gemm, p.scale_relu, nt);
                    else
                        store_row16_i8<EPI_PASSTHROUGH>(crow, 16 * (int)q, KOUT, vec_ok, acc, p.scale_gemm, p.scale_relu, nt);
                }
            }
        }
    }
};

template <int DT>
__global__ __launch_bounds__(256, 2) void conv_stem_kernel(const ConvStemArgs p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t ckx_smem[];
    ConvStem<DT>::run(p, ckx_smem);
}

// (conv_stem.hip)
hipError_t launch_conv_stem(int dt, const ConvStemArgs& a, hipStream_t s);

} // namespace ckx
