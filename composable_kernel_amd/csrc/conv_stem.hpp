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
// Algorithmic traffic is the output (N x 112 x 112 x 64) by far: the layer is bound by HBM writes. Measured at N = 256
// (timing-only builds, fp16): 148 us; 86 without the input loads (the stores alone, at the write rate of the part);
// 78 without the stores; 59 without either (MFMAs at 28 per 16 pixels, LDS, barriers). Reads issued into a memory system
// that is saturated with writes come back late; a variant with a dedicated copy wave per workgroup and two band buffers
// (no wave both loads and stores) measured the same for fp16 and worse for int8, and was not kept.
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
    // (the padded weight matrix passes through the same LDS first: 64 rows x 7 (8) filter rows x 32 elements)
    __host__ __device__ static int lds_bytes(int Wo)
    {
        const int band = ROWS * slot_bytes(Wo), weights = KOUT * (DT == DT_I8 ? 8 : 7) * 32 * ES;
        return band > weights ? band : weights;
    }

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

        // ---- the weights as B fragments. First the padded [64][KP] matrix in LDS, K order (y, x', c') with zeros at
        // x' = 7, c' = 3 (and filter row 7 for int8), filled by all threads with consecutive addresses; then N tile t,
        // k-step ks: lane (r, q) takes the 16 bytes at K element ks * KE + q * VE of LDS-order row 16 t + r, which is
        // output channel b_row_to_col(16 t + r). (Fetched from global memory element by element under the validity
        // test, a lane's 224 loads each took a round trip.)
        constexpr int KP = (DT == DT_I8 ? 8 : 7) * 32, KE = DT == DT_I8 ? 64 : 32, VE = 16 / ES;
        {
            elem_t* wl = reinterpret_cast<elem_t*>(smem);
#pragma unroll 8
            for(int i = tid; i < KOUT * KP; i += NTHR)
            {
                const int n = i / KP, k = i - n * KP;
                const int y = k >> 5, x = (k >> 2) & 7, c = k & 3;
                const bool ok = y < Y && x < X && c < C;
                const elem_t v = wei[((n * Y + (ok ? y : 0)) * X + (ok ? x : 0)) * C + (ok ? c : 0)];
                wl[i]          = ok ? v : (elem_t)0;
            }
        }
        __syncthreads();
        i32x4 bfr[4][NKS];
#pragma unroll
        for(int t = 0; t < 4; ++t)
        {
            const int n = (int)b_row_to_col((uint32_t)(16 * t) + r);
#pragma unroll
            for(int ks = 0; ks < NKS; ++ks)
                bfr[t][ks] = *reinterpret_cast<const i32x4*>(smem + (n * KP + ks * KE + (int)q * VE) * ES);
        }
        // (the band copy below starts behind a barrier)
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
            // ---- copy the band: padded pixel slot pp of LDS row rr <- input pixel (hi0 + rr, pp - PAD), zeros outside.
            // A thread takes one pixel column of all the band's rows: every load is requested before the first LDS write
            // (row by row, each write behind its own load, the copy took ROWS memory round trips per band: 219 us for the
            // layer against 157).
            const int npx = slot / PX;
            __syncthreads(); // (every wave is done with the previous band)
            for(int pp = tid; pp < npx; pp += NTHR)
            {
                const int wi     = pp - PAD;
                const bool wi_ok = wi >= 0 && wi < p.Wi;
                struct __attribute__((packed, aligned(ES))) px3
                {
                    elem_t c[3];
                };
                px3 v[ROWS];
#pragma unroll
                for(int rr = 0; rr < ROWS; ++rr)
                {
                    const int hi  = hi0 + rr;
                    const bool ok = wi_ok && hi >= 0 && hi < p.Hi;
                    const px3* src = reinterpret_cast<const px3*>(in + ((size_t)(n * p.Hi + (ok ? hi : 0)) * p.Wi + (ok ? wi : 0)) * C);
                    v[rr]          = ok ? *src : px3{{(elem_t)0, (elem_t)0, (elem_t)0}};
                }
#pragma unroll
                for(int rr = 0; rr < ROWS; ++rr)
                {
                    typedef elem_t ex4 __attribute__((ext_vector_type(4)));
                    *reinterpret_cast<ex4*>(smem + rr * slot + pp * PX) = ex4{v[rr].c[0], v[rr].c[1], v[rr].c[2], (elem_t)0};
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
__global__ __launch_bounds__(256, DT == DT_I8 ? 3 : 2) void conv_stem_kernel(const ConvStemArgs p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t ckx_smem[];
    ConvStem<DT>::run(p, ckx_smem);
}

// (conv_stem.hip)
hipError_t launch_conv_stem(int dt, const ConvStemArgs& a, hipStream_t s);

} // namespace ckx
