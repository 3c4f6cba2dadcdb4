// Weight-stationary pointwise (1x1) conv2d forward for gfx950, fp16 and int8, NHWC / KYXC / NHWK: layers
// with a short reduction and a large output (ResNet projection shortcuts: C = 256 -> K = 512, stride 2),
// where the tile kernel runs four K tiles per C tile and then sits in a workgroup-wide epilogue whose
// stores the next tile's first wait has to drain.
//
// Takes the place of the same reference kernel as the tile kernel
// (DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K,
// device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720, with its Filter1x1Pad0 / Filter1x1Stride1Pad0
// specialisations :124-220) for the shapes it covers:
//   Y = X = 1, no padding, any stride; C * element size = 256 or 512 bytes; K a multiple of 512.
//
//  * The weights never touch LDS. A workgroup is 8 waves and covers 512 output channels; wave w keeps
//    the whole [64 channels x C] weight slice of its channels in REGISTERS for the life of the workgroup
//    (4 MFMA tiles x KS k-steps x 4 VGPRs: 128 of them at C * es = 512 bytes).
//  * Pixels stream through an LDS RING of bands (16 * MT pixels x one pixel's channels per slot, 9 slots of
//    16 KB), filled by direct global->LDS loads 7 bands ahead of the band being multiplied: HBM latency is
//    out of the loop, and the one barrier per band is the only place the waves meet.
//  * A wave multiplies every band by its weight slice: per 16-pixel tile KS fragment reads feed 4 * KS
//    MFMAs. The fragment registers are a single set refilled in place: the read of the NEXT tile's k-step
//    goes out right after the MFMAs that consumed the current one (a full tile of lead).
//  * Each wave converts and stores its own 16 pixels x 64 channels as soon as a tile is done (two
//    accumulator sets alternate), so stores from some waves overlap the MFMAs of the others, and no wave
//    ever waits for them: the only vmcnt wait counts direct loads issued 6 bands later or more.
//  * 16-byte chunks of a pixel are swizzled with the pixel's position in its 16-pixel tile
//    (chunk ^ (row & 15)): the 16 rows of a fragment read cover all 64 banks.
//  * D^T = B_frag x A_frag with the weight rows taken in permuted order (as the tile kernel permutes them in
//    LDS), so a lane owns 16 consecutive channels of one pixel: 16-byte stores, no trip through LDS.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct ConvPointwiseArgs
{
    const void* in;
    const void* wei;
    void* out;
    uint32_t in_bytes;
    int M;    // N * Ho * Wo output pixels
    int Kout; // output channels
    int Hi, Wi, Wo, HoWo, sH, sW;
    MagicDiv div_howo, div_wo;
    int epi; // fp16: EPI_PASSTHROUGH, EPI_ADD_RELU (bias row); int8: EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND,
             // EPI_MUL2_CLAMP / EPI_RELU_MUL2_CLAMP (one requant scale per output channel)
    const void* bias; // [Kout]: fp16 bias (fp16 kernels), fp32 requant scales (the int8 per-channel variant)
    float scale_gemm, scale_relu;
    int nt_store; // stream the output past L2 (outputs too large to be re-read from cache)
};

// KS: MFMA k-steps per pixel (C * element size / 64 bytes); MT: 16-pixel tiles per band;
// FUSED: fp16 -- the bias + ReLU epilogue is compiled in; int8 -- the per-channel requant epilogue
// (Activation_Mul2_Clamp) INSTEAD of the per-tensor ones
template <int DT, int KS, int MT, bool FUSED>
struct ConvPointwise
{
    static constexpr int ES   = DT == DT_I8 ? 1 : 2;
    static constexpr int RB   = 64 * KS; // bytes of one pixel
    static constexpr int CPR  = RB / 16; // 16-byte chunks per pixel
    static constexpr int MB   = 16 * MT; // pixels per band
    static constexpr int SLOT = MB * RB;
    static constexpr int D    = 9;       // ring slots; D - 2 bands are in flight ahead of the one being multiplied
    static constexpr int LUT  = DT == DT_I8 ? 256 : 0; // table of the rounded requant epilogue, behind the ring
    static constexpr int LDS  = D * SLOT + LUT;
    static constexpr int NW   = 8;
    static constexpr int NT   = 64 * NW;
    static constexpr int LPW  = SLOT / 1024 / NW; // direct loads per wave and band
    static constexpr int NWG  = 64 * NW;          // output channels per workgroup
    static_assert(KS == 4 || KS == 8, "pixels of 256 or 512 bytes");
    static_assert(DT == DT_F16 || DT == DT_I8, "fp16 (optionally bias + ReLU) or int8 (per-tensor or per-channel requant)");
    static_assert(SLOT % (1024 * NW) == 0 && LPW >= 1 && LPW <= KS, "every wave issues the same number of loads");
    static_assert(LDS <= 160 * 1024 && (D - 3) * LPW < 64, "ring fits the LDS, vmcnt is a 6-bit counter");
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;

    __device__ static __forceinline__ void run(const ConvPointwiseArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
        const __amdgpu_buffer_rsrc_t rsrc_in = make_rsrc(p.in, p.in_bytes);
        if constexpr(DT == DT_I8)
        {
            // table of the rounded requant epilogue (visible after the first band's barrier)
            if(p.epi == EPI_REQUANT_RND)
                requant_lut_fill(smem + D * SLOT, p.scale_relu, (int)threadIdx.x, 512);
        }

        // ---- the wave's weight slice. A lane ends up with MFMA rows 4q..4q+3 of each of the four tiles (q = lane / 16);
        // which channel sits in which MFMA row is free, and chosen so that a lane's values are whole 16-byte runs of
        // one pixel and the four lanes of a pixel write 64 contiguous bytes per store instruction:
        //   int8: tile t, row j <- channel 16 * (j / 4) + 4 * t + j % 4 (16 consecutive channels per lane);
        //   fp16: tile t, row j <- channel 32 * (t / 2) + 8 * (j / 4) + 4 * (t % 2) + j % 4 (two runs of 8)
        const int n_wave = (int)blockIdx.y * NWG + wave * 64;
        i32x4 bw[4][KS];
#pragma unroll
        for(int t = 0; t < 4; ++t)
        {
            const int n = ES == 1 ? n_wave + 16 * (int)(frow >> 2) + 4 * t + (int)(frow & 3)
                                  : n_wave + 32 * (t >> 1) + 8 * (int)(frow >> 2) + 4 * (t & 1) + (int)(frow & 3);
            const uint8_t* wrow = reinterpret_cast<const uint8_t*>(p.wei) + (size_t)n * RB + 16 * fq;
#pragma unroll
            for(int ks = 0; ks < KS; ++ks)
                bw[t][ks] = *reinterpret_cast<const i32x4*>(wrow + 64 * ks);
        }
        // the lane's output channels: int8 16 consecutive ones (16 bytes; four lanes write 64 contiguous bytes of a
        // pixel), fp16 two runs of 8, at n0 and n0 + 32 (each store instruction again 64 contiguous bytes per pixel)
        const int n0 = n_wave + (ES == 1 ? 16 : 8) * (int)fq;
        f16x8 bias_lo = {0, 0, 0, 0, 0, 0, 0, 0}, bias_hi = bias_lo;
        float chsc[DT == DT_I8 && FUSED ? 16 : 1]; // the requant scales of the lane's 16 channels
        if constexpr(DT == DT_I8 && FUSED)
        {
#pragma unroll
            for(int e = 0; e < 16; ++e)
                chsc[e] = reinterpret_cast<const float*>(p.bias)[n0 + e];
        }
        else if constexpr(FUSED)
        {
            bias_lo = *reinterpret_cast<const f16x8*>(reinterpret_cast<const _Float16*>(p.bias) + n0);
            bias_hi = *reinterpret_cast<const f16x8*>(reinterpret_cast<const _Float16*>(p.bias) + n0 + 32);
        }

        // ---- fragment addresses: row frow of a tile, chunk (4 * ks + fq) ^ frow. The k-step enters as an XOR on
        // address bits 6-7 (four lane constants) and, for 512-byte pixels, + 256 bytes (offset field)
        uint32_t lk[4];
        {
            const uint32_t l0 = frow * RB + (((fq ^ (frow & 3u)) + (frow & 12u)) << 4);
#pragma unroll
            for(int k = 0; k < 4; ++k)
                lk[k] = l0 ^ ((uint32_t)k << 6);
        }

        // ---- direct loads: load li of a wave covers chunk positions ((wave * LPW + li) * 64 + lane) of the slot;
        // position (row, pos) receives global chunk pos ^ (row & 15) of that pixel
        uint32_t ld_row[LPW], ld_chunk[LPW];
#pragma unroll
        for(int li = 0; li < LPW; ++li)
        {
            const uint32_t idx = (uint32_t)((wave * LPW + li) * 64 + lane);
            ld_row[li]         = idx / CPR;
            ld_chunk[li]       = ((idx % CPR) ^ (ld_row[li] & 15u)) << 4;
        }
        const long nb_total = ((long)p.M + MB - 1) / MB;
        const int band_lo   = (int)(nb_total * (long)blockIdx.x / (long)gridDim.x);
        const int band_hi   = (int)(nb_total * ((long)blockIdx.x + 1) / (long)gridDim.x);
        auto issue_load = [&](int band, int slot, int li) {
            const uint32_t m   = (uint32_t)band * MB + ld_row[li];
            const bool ok      = band < band_hi && m < (uint32_t)p.M;
            const uint32_t img = magic_div(m, p.div_howo);
            const uint32_t rem = m - img * (uint32_t)p.HoWo;
            const uint32_t ho  = magic_div(rem, p.div_wo);
            const uint32_t wo  = rem - ho * (uint32_t)p.Wo;
            const uint32_t pix = (img * (uint32_t)p.Hi + ho * (uint32_t)p.sH) * (uint32_t)p.Wi + wo * (uint32_t)p.sW;
            const uint32_t voff = (pix * RB + ld_chunk[li]) | (ok ? 0u : kOutOfRange);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rsrc_in, (lds_ptr_t)(smem + (size_t)slot * SLOT + (size_t)(wave * LPW + li) * 1024), 16, voff, 0, 0, 0);
        };
        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };

        int ld_band = band_lo, ld_slot = 0;
        for(int i = 0; i < D - 1; ++i)
        {
#pragma unroll
            for(int li = 0; li < LPW; ++li)
                issue_load(ld_band, ld_slot, li);
            ++ld_band;
            ld_slot = ld_slot + 1 == D ? 0 : ld_slot + 1;
        }
        // the first band has landed (the weight loads are older still)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 2) * LPW) : "memory");
        barrier();

        uint32_t cur[4], nxt[4];
#pragma unroll
        for(int k = 0; k < 4; ++k)
            cur[k] = nxt[k] = smem_lds + lk[k];
        i32x4 af[KS];
        static_for<KS>([&](auto ks_c) {
            constexpr int ks = decltype(ks_c)::value;
            af[ks]           = lds_read_b128<(ks >> 2) * 256>(cur[ks & 3]);
        });
        acc_t acc[2][4];
        const bool nt = p.nt_store != 0;

        auto run_bands = [&](auto epi_c) {
            constexpr int EPI = decltype(epi_c)::value;
            int slot = 0;
            for(int band = band_lo; band < band_hi; ++band)
            {
                static_for<MT>([&](auto t_c) {
                    constexpr int t     = decltype(t_c)::value;
                    constexpr bool last = t == MT - 1;
                    if constexpr(last)
                    {
                        // The next band has landed (this wave's share): direct loads retire in order, so at
                        // most the loads of the D - 3 bands behind it may be outstanding. Stores share the
                        // counter; they can only make this wait longer, never too short. Past the barrier every
                        // wave has every fragment of the PREVIOUS band in registers: its slot is refilled.
                        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 3) * LPW) : "memory");
                        barrier();
                        slot = slot + 1 == D ? 0 : slot + 1;
#pragma unroll
                        for(int k = 0; k < 4; ++k)
                            nxt[k] = smem_lds + (uint32_t)(slot * SLOT) + lk[k];
                    }
                    static_for<KS>([&](auto ks_c) {
                        constexpr int ks = decltype(ks_c)::value;
                        // fragment ks of this tile: KS - 1 reads were issued after it
                        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(KS - 1));
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for(int tn = 0; tn < 4; ++tn)
                        {
                            const acc_t c = ks == 0 ? acc_t{0, 0, 0, 0} : acc[t & 1][tn];
                            if constexpr(DT == DT_I8)
                                acc[t & 1][tn] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bw[tn][ks], af[ks], c, 0, 0, 0);
                            else
                                acc[t & 1][tn] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    __builtin_bit_cast(f16x8, bw[tn][ks]), __builtin_bit_cast(f16x8, af[ks]), c, 0, 0, 0);
                        }
                        // the same k-step of the next tile (of the next band after the last tile) into the
                        // registers just consumed
                        if constexpr(last)
                            af[ks] = lds_read_b128<(ks >> 2) * 256>(nxt[ks & 3]);
                        else
                            af[ks] = lds_read_b128<(t + 1) * 16 * RB + (ks >> 2) * 256>(cur[ks & 3]);
                        if constexpr(last && ks < LPW)
                            issue_load(ld_band, ld_slot, ks);
                        __builtin_amdgcn_sched_barrier(0);
                    });

                    // ---- this tile's 16 pixels x the wave's 64 channels: 16 consecutive channels per lane
                    // (K is a multiple of 512 and the output 16-byte aligned: whole vectors, no tail)
                    const int m = band * MB + 16 * t + (int)frow;
                    if(m < p.M)
                    {
                        if constexpr(DT == DT_I8)
                        {
                            i32x4 pk;
                            if constexpr(EPI == EPI_MUL2_CLAMP || EPI == EPI_RELU_MUL2_CLAMP)
                            {
#pragma unroll
                                for(int tn = 0; tn < 4; ++tn)
                                    pk[tn] = pack4_low_bytes(
                                        mul2_clamp(acc[t & 1][tn][0], chsc[(4 * tn) % (FUSED ? 16 : 1)], EPI == EPI_RELU_MUL2_CLAMP),
                                        mul2_clamp(acc[t & 1][tn][1], chsc[(4 * tn + 1) % (FUSED ? 16 : 1)], EPI == EPI_RELU_MUL2_CLAMP),
                                        mul2_clamp(acc[t & 1][tn][2], chsc[(4 * tn + 2) % (FUSED ? 16 : 1)], EPI == EPI_RELU_MUL2_CLAMP),
                                        mul2_clamp(acc[t & 1][tn][3], chsc[(4 * tn + 3) % (FUSED ? 16 : 1)], EPI == EPI_RELU_MUL2_CLAMP));
                            }
                            else if constexpr(EPI == EPI_REQUANT_RND)
                            {
                                const i32x4 v[4] = {acc[t & 1][0], acc[t & 1][1], acc[t & 1][2], acc[t & 1][3]};
                                int b[16];
                                requant_lut<4>(v, p.scale_gemm, smem_lds + (uint32_t)(D * SLOT), b);
#pragma unroll
                                for(int tn = 0; tn < 4; ++tn)
                                    pk[tn] = pack4_low_bytes(b[4 * tn], b[4 * tn + 1], b[4 * tn + 2], b[4 * tn + 3]);
                            }
                            else
                            {
#pragma unroll
                                for(int tn = 0; tn < 4; ++tn)
                                    pk[tn] = pack4_low_bytes(epilogue_i8<EPI>(acc[t & 1][tn][0], p.scale_gemm, p.scale_relu),
                                                             epilogue_i8<EPI>(acc[t & 1][tn][1], p.scale_gemm, p.scale_relu),
                                                             epilogue_i8<EPI>(acc[t & 1][tn][2], p.scale_gemm, p.scale_relu),
                                                             epilogue_i8<EPI>(acc[t & 1][tn][3], p.scale_gemm, p.scale_relu));
                            }
                            store_vec(reinterpret_cast<i32x4*>(reinterpret_cast<int8_t*>(p.out) + (size_t)m * p.Kout + n0), pk, nt);
                        }
                        else
                        {
                            f16x8 o[2];
#pragma unroll
                            for(int tn = 0; tn < 4; ++tn)
#pragma unroll
                                for(int j = 0; j < 4; ++j)
                                {
                                    float v = acc[t & 1][tn][j];
                                    if constexpr(EPI == EPI_ADD_RELU)
                                    {
                                        v += (float)(tn < 2 ? bias_lo[(tn & 1) * 4 + j] : bias_hi[(tn & 1) * 4 + j]);
                                        v = v > 0.0f ? v : 0.0f;
                                    }
                                    o[tn >> 1][(tn & 1) * 4 + j] = (_Float16)v;
                                }
                            f16x8* dst = reinterpret_cast<f16x8*>(reinterpret_cast<_Float16*>(p.out) + (size_t)m * p.Kout + n0);
                            store_vec(dst, o[0], nt);
                            store_vec(dst + 4, o[1], nt);
                        }
                    }
                });
#pragma unroll
                for(int k = 0; k < 4; ++k)
                    cur[k] = nxt[k];
                ++ld_band;
                ld_slot = ld_slot + 1 == D ? 0 : ld_slot + 1;
            }
        };
        if constexpr(DT == DT_I8 && FUSED)
        {
            if(p.epi == EPI_RELU_MUL2_CLAMP)
                run_bands(std::integral_constant<int, EPI_RELU_MUL2_CLAMP>{});
            else
                run_bands(std::integral_constant<int, EPI_MUL2_CLAMP>{});
        }
        else if constexpr(DT == DT_I8)
        {
            if(p.epi == EPI_REQUANT_RND)
                run_bands(std::integral_constant<int, EPI_REQUANT_RND>{});
            else if(p.epi == EPI_REQUANT_CK)
                run_bands(std::integral_constant<int, EPI_REQUANT_CK>{});
            else
                run_bands(std::integral_constant<int, EPI_PASSTHROUGH>{});
        }
        else if constexpr(FUSED)
            run_bands(std::integral_constant<int, EPI_ADD_RELU>{});
        else
            run_bands(std::integral_constant<int, EPI_PASSTHROUGH>{});
        // trailing (zero-fill) loads still target this workgroup's LDS, trailing reads its registers
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
};

template <int DT, int KS, int MT, bool FUSED>
__global__ __launch_bounds__(512) void conv_pointwise_kernel(const ConvPointwiseArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_pointwise_smem[];
    ConvPointwise<DT, KS, MT, FUSED>::run(p, ckx_pointwise_smem);
}

// conv_pointwise.hip: dt = DT_I8 / DT_F16, pixel_bytes = C * element size (256 or 512), fused = fp16 bias + ReLU
hipError_t launch_conv_pointwise(int dt, int pixel_bytes, bool fused, const ConvPointwiseArgs& a, hipStream_t s);

} // namespace ckx
