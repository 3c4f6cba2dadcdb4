// Input-patch conv2d forward for gfx950, fp16, NHWC / KYXC / NHWK: the 3x3-class layers with few
// channels (ResNet conv2_x: C = 64, K = 64, 56 x 56), where the implicit-GEMM tile kernel re-reads
// every input pixel once per filter tap out of L2 and is bound by that.
//
// Takes the place of the same reference kernel as the tile kernel
// (DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K,
// device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720) for the shapes it covers:
//   C * 2 bytes = 128 (one pixel = one 128-byte LDS row = one tap's K tile), K = 64,
//   Y x X taps, stride 1, dilation 1, Wo = 8 * MTW <= 56, Wo + X - 1 <= 64.
//
//  * A workgroup (4 waves) owns whole images and walks them in bands of 4 output rows. The
//    input rows a band needs (4 + Y - 1) live in LDS in a RING of 10 rows x 64 pixels x 128 B;
//    while band b is multiplied, the 4 new rows of band b + 1 are fetched into the ring slots
//    that band b - 1 has finished with. Every input pixel is read from memory ONCE.
//  * All Y * X * 64 weight rows (72 KB) are LDS-resident for the life of the workgroup.
//  * The A fragment of tap (y, x) for 16 consecutive output pixels is the patch shifted by
//    (y rows, x pixels): the same 128-byte rows, another base address. A lane keeps one
//    precomputed byte offset per (M tile, x) and one per (M tile, y): a fragment address is one add.
//  * 16-byte chunks are swizzled by the patch COLUMN (chunk ^ (col & 7)), so the 16 pixels of a
//    fragment read spread over the banks exactly as the 16 rows of a GEMM fragment do.
//  * 2 x 2 waves: a wave multiplies 16 * MTW pixels x 32 output channels; D^T = B_frag x A_frag with
//    the weight rows permuted in LDS so that a lane ends up with 8 consecutive channels of one
//    pixel: one 16-byte store, no trip through LDS.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct ConvPatchArgs
{
    const void* in;
    const void* wei;
    void* out;
    uint32_t in_bytes, wei_bytes;
    int N, Hi, Wi, Ho, Wo;
    int pT, pL;
    int nbands; // ceil(Ho / 4)
    MagicDiv div_wo;
    int epi; // EPI_PASSTHROUGH, EPI_ADD_RELU, EPI_ADD_RELU_ADD
    const void* bias; // [64] fp16
    const void* resi; // NHWK fp16
};

// FUSED: the add / ReLU epilogues (bias, residual) are compiled in; the plain instantiation keeps
// their registers free
template <int MTW, int Y, int X, bool FUSED>
struct ConvPatch
{
    static constexpr int TH     = 4;                // output rows per band
    static constexpr int RING   = 2 * TH + 2;       // ring rows (Y <= 3)
    static constexpr int PITCH  = 64;               // pixels per ring row
    static constexpr int PXB    = 128;              // bytes per pixel (C * 2)
    static constexpr int KO     = 64;               // output channels
    static constexpr int TAPS   = Y * X;
    static constexpr int RING_BYTES = RING * PITCH * PXB;
    static constexpr int WEI_BYTES  = TAPS * KO * PXB;
    static constexpr int LDS        = RING_BYTES + WEI_BYTES;
    static constexpr int NT         = 256;
    static constexpr int NEED_ROWS  = TH + Y - 1;   // input rows of one band
    static_assert(Y >= 1 && Y <= 3 && X >= 1 && X <= 3 && MTW >= 1 && MTW <= 7, "covered shapes");

    __device__ static __forceinline__ void run(const ConvPatchArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int wm = wave >> 1, wn = wave & 1;
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        uint8_t* ring = smem;
        uint8_t* wlds = smem + RING_BYTES;

        const __amdgpu_buffer_rsrc_t rsrc_in  = make_rsrc(p.in, p.in_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_wei = make_rsrc(p.wei, p.wei_bytes);

        // ---- weights: LDS row tap*64 + r holds output channel w_row_to_ch(r), swizzled by r & 7
        {
            const uint32_t rl  = (uint32_t)(lane >> 3);  // row within the 8-row block = its swizzle key
            const uint32_t pos = (uint32_t)(lane & 7);
            for(int k = wave; k < TAPS * 8; k += 4)
            {
                const uint32_t tap = (uint32_t)k >> 3;
                const uint32_t r   = (((uint32_t)k & 7u) << 3) + rl; // 0..63
                // within a 32-row group, row 16j + 4q + i holds channel 8q + 4j + i
                const uint32_t ch = (r & ~31u) | (((r >> 2) & 3u) << 3) | (((r >> 4) & 1u) << 2) | (r & 3u);
                const uint32_t voff = (ch * TAPS + tap) * PXB + ((pos ^ rl) << 4);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_wei, (lds_ptr_t)(wlds + (size_t)k * 1024), 16, voff, 0,
                                                         0, 0);
            }
        }

        // ---- per-lane constants of the wave's M tiles -----------------------------------
        uint32_t coff[MTW][X]; // (col * 128 + swizzled chunk of k-step 0) for tap column x
        uint32_t rout[MTW];    // output row of the lane's pixel within the band (0..3)
        uint32_t ooff[MTW];    // byte offset of the lane's 8 outputs relative to the band
#pragma unroll
        for(int t = 0; t < MTW; ++t)
        {
            const uint32_t q = (uint32_t)((wm * MTW + t) * 16) + frow;
            const uint32_t r = magic_div(q, p.div_wo);
            const uint32_t w = q - r * (uint32_t)p.Wo;
            rout[t]          = r;
            ooff[t]          = ((r * (uint32_t)p.Wo + w) * KO + (uint32_t)(32 * wn) + 8u * fq) * 2u;
#pragma unroll
            for(int x = 0; x < X; ++x)
            {
                const uint32_t cc = w + (uint32_t)x;
                coff[t][x]        = cc * PXB + ((fq ^ (cc & 7u)) << 4);
            }
        }
        // fused add / ReLU epilogues: the lane's 8 bias values once, its residual values band by band
        const bool has_resi = FUSED && p.epi == EPI_ADD_RELU_ADD;
        f16x8 bias8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr(FUSED)
            bias8 = *reinterpret_cast<const f16x8*>(reinterpret_cast<const _Float16*>(p.bias) + 32 * wn + 8 * (int)fq);
        f16x8 resi8[FUSED ? MTW : 1];
#pragma unroll
        for(int t = 0; t < (FUSED ? MTW : 1); ++t)
            resi8[t] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};

        uint32_t boff[2]; // weight fragment of n-tile j, k-step 0, tap 0
#pragma unroll
        for(int j = 0; j < 2; ++j)
            boff[j] = (uint32_t)(32 * wn + 16 * j + (int)frow) * PXB + ((fq ^ (frow & 7u)) << 4);

        // ---- input rows -> ring: block k = (row j, 8-pixel column group cg) ------------------
        // lane: patch column 8*cg + lane/8, LDS chunk position lane%8 <- global chunk pos ^ (col & 7)
        auto load_block = [&](int n, int j, int cg) {
            const int cc = 8 * cg + (lane >> 3);
            const int wi = cc - p.pL, hi = j - p.pT;
            const bool ok = (uint32_t)hi < (uint32_t)p.Hi && (uint32_t)wi < (uint32_t)p.Wi && n < p.N;
            const uint32_t chunk = (uint32_t)(lane & 7) ^ (uint32_t)(lane >> 3);
            const uint32_t voff =
                ((uint32_t)((n * p.Hi + hi) * p.Wi + wi) * PXB + (chunk << 4)) | (ok ? 0u : kOutOfRange);
            const int slot = j % RING;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_ptr_t)(ring + (size_t)(slot * PITCH + 8 * cg) * PXB),
                                                     16, voff, 0, 0, 0);
        };

        f32x4 acc[MTW][2];
#pragma unroll
        for(int t = 0; t < MTW; ++t)
            acc[t][0] = acc[t][1] = f32x4{0, 0, 0, 0};

        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };

        uint32_t roff[MTW][Y]; // ring byte offset of (M tile's output row + y) for the current band
        i32x4 af[2][MTW], bf[2][2];
        for(int n = (int)blockIdx.x; n < p.N; n += (int)gridDim.x)
        {
            // rows of the first band (every wave has passed the barrier that ended the previous image)
            for(int k = wave; k < NEED_ROWS * 8; k += 4)
                load_block(n, k >> 3, k & 7);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            barrier();

            for(int b = 0; b < p.nbands; ++b)
            {
                const int j0 = TH * b; // first ring row index (before the modulo) of this band
                if(b == 0)
                {
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
#pragma unroll
                        for(int y = 0; y < Y; ++y)
                            roff[t][y] = (rout[t] + (uint32_t)y) * (PITCH * PXB);
                }

                // fragment r of k-step s = (tap, half): r = 0, 1 the two weight tiles, then the M tiles
                // in the order in which the MFMAs use them
                auto read_one = [&](int s, int r) {
                    const int buf = s & 1, tap = s >> 1, ks = s & 1, y = tap / X, x = tap % X;
                    if(r < 2)
                        bf[buf][r] = *reinterpret_cast<const i32x4*>(wlds + tap * (KO * PXB) +
                                                                     (boff[r] ^ (uint32_t)(ks * 64)));
                    else
                        af[buf][r - 2] = *reinterpret_cast<const i32x4*>(ring + roff[r - 2][y] +
                                                                         (coff[r - 2][x] ^ (uint32_t)(ks * 64)));
                };
                auto mfma_pair = [&](int s, int t) {
                    const int buf = s & 1;
#pragma unroll
                    for(int j = 0; j < 2; ++j)
                        acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bf[buf][j]),
                                                                        __builtin_bit_cast(f16x8, af[buf][t]),
                                                                        acc[t][j], 0, 0, 0);
                };

                if(b == 0)
                {
#pragma unroll
                    for(int r = 0; r < MTW + 2; ++r)
                        read_one(0, r);
                }
                // residual values of this band: plain loads, issued before the band's direct loads and
                // waited for with them (a load issued after the stores would have to wait for those)
                if constexpr(FUSED)
                  if(has_resi)
                {
                    const uint8_t* resi_band = reinterpret_cast<const uint8_t*>(p.resi) +
                                               ((size_t)n * p.Ho + (size_t)TH * b) * p.Wo * (KO * sizeof(_Float16));
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
                        if(TH * b + (int)rout[t] < p.Ho)
                            resi8[FUSED ? t : 0] = *reinterpret_cast<const f16x8*>(resi_band + ooff[t]);
                }
                // One k-step = MTW groups pinned in source order: [reads of the NEXT k-step, spread over
                // the first groups and finished two groups early] [one direct load of the next band's
                // rows] [the 2 MFMAs of one M tile]. With one wave per SIMD nothing else hides the
                // issue slots of the reads, so they go between the MFMAs.
                constexpr int NR = MTW + 2, RG = MTW > 2 ? MTW - 2 : MTW;
#pragma unroll
                for(int s = 0; s < 2 * TAPS; ++s)
                {
#pragma unroll
                    for(int g = 0; g < MTW; ++g)
                    {
                        if(s + 1 < 2 * TAPS)
                        {
#pragma unroll
                            for(int r = (g < RG ? g : RG) * NR / RG; r < (g + 1 < RG ? g + 1 : RG) * NR / RG; ++r)
                                read_one(s + 1, r);
                        }
                        // the 4 new input rows of the next band: 32 blocks, 8 per wave, one per k-step
                        if(s < 8 && g == MTW - 1)
                        {
                            const int k = wave + 4 * s;
                            load_block(n, j0 + NEED_ROWS + (k >> 3), k & 7);
                        }
                        mfma_pair(s, g);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }

                // the next band's rows have landed (this wave's share) before the stores go out:
                // stores share the counter with loads and are not ordered against them
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                // every wave is through with this band's rows, and the next band's rows are visible:
                // its first fragments are read under the epilogue
                barrier();
                if(b + 1 < p.nbands)
                {
                    const int j1 = j0 + TH;
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
#pragma unroll
                        for(int y = 0; y < Y; ++y)
                        {
                            uint32_t sl = (uint32_t)(j1 % RING) + rout[t] + (uint32_t)y;
                            sl          = sl >= (uint32_t)RING ? sl - RING : sl;
                            roff[t][y]  = sl * (PITCH * PXB);
                        }
#pragma unroll
                    for(int r = 0; r < MTW + 2; ++r)
                        read_one(0, r);
                }

                // ---- epilogue: 8 consecutive channels of one pixel per lane and M tile ----------
                _Float16* out_band = reinterpret_cast<_Float16*>(p.out) + ((size_t)n * p.Ho + (size_t)TH * b) * p.Wo * KO;
#pragma unroll
                for(int t = 0; t < MTW; ++t)
                {
                    if(TH * b + (int)rout[t] < p.Ho)
                    {
                        f16x8 o;
#pragma unroll
                        for(int i = 0; i < 4; ++i)
                        {
                            float v0 = acc[t][0][i], v1 = acc[t][1][i];
                            if constexpr(FUSED)
                            {
                                v0 = epi_f16_value(p.epi, v0, (float)bias8[i], (float)resi8[t][i]);
                                v1 = epi_f16_value(p.epi, v1, (float)bias8[4 + i], (float)resi8[t][4 + i]);
                            }
                            o[i]     = (_Float16)v0;
                            o[4 + i] = (_Float16)v1;
                        }
                        *reinterpret_cast<f16x8*>(reinterpret_cast<uint8_t*>(out_band) + ooff[t]) = o;
                    }
                    acc[t][0] = acc[t][1] = f32x4{0, 0, 0, 0};
                }
            }
            barrier(); // the ring is free for the next image's first rows
        }
        // the weight loads of a workgroup that got no image still target its LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
};

template <int MTW, int Y, int X, bool FUSED>
__global__ __launch_bounds__(256) void conv_patch_kernel(const ConvPatchArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_patch_smem[];
    ConvPatch<MTW, Y, X, FUSED>::run(p, ckx_patch_smem);
}

} // namespace ckx
