// Input-patch conv2d forward for 3 x 3 layers with 128 input and 128 output channels (ResNet conv3_x, 28 x 28), fp16 and
// int8, NHWC / KYXC / NHWK: the arrangement of conv_patch.hpp (a workgroup owns whole images, input rows in an LDS ring,
// weights in AccVGPRs, every fragment address a fixed register plus an immediate) for a layer whose weights are four
// times as large -- 288 KB in fp16: no LDS holds them and no four waves' registers do.
//
// Takes the place of the same reference kernel as the tile kernel
// (DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K, device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720)
// for C = 128, K = 128, 3 x 3 taps, stride 1, dilation 1, Wo = 28.
//
//  * FOUR waves, one per SIMD, multiply the SAME pixels and split the OUTPUT CHANNELS: wave w owns channels 32 w .. 32 w + 31
//    and keeps their 9 taps x 128 input channels as 72 (fp16) / 36 (int8) MFMA operand fragments in registers -- fp16: 60 of
//    them in 240 AccVGPRs and the last 12 in VGPRs (all 256 AccVGPRs would leave the allocator nothing to move a value
//    through), int8: 144 AccVGPRs -- beside 14 accumulator tiles, 7 pixel fragments and 21 read addresses.
//  * A band of 4 output rows x 28 pixels is 7 M tiles for every wave; a pixel fragment read feeds two MFMAs. That ratio is
//    what decides the arrangement: a wave-wide ds_read_b128 occupies the CU's LDS pipe for 8 cycles, an MFMA a SIMD's
//    matrix core for 16, so four waves at one read per two MFMAs keep the LDS pipe as busy as the matrix cores. EIGHT
//    waves of 16 channels (NW_ = 8: 36 fragments per wave, 128 AccVGPRs + 16 VGPRs of the 128 + 128 a wave then has) read
//    one fragment per MFMA: measured 60.0 against 50.2 us in fp16 and 33.0 against 29.1 in int8 at N = 256, and timing-only
//    builds of that form took 54 us with a seventh of the MFMAs, 49 us with a seventh of the reads -- bound by the LDS.
//  * A ring row is 4 (fp16) / 2 (int8) planes of 32 pixels x 64 bytes; the k-step, the tap row and the band's position in
//    the ring are offsets, the tap column selects one of three per-lane registers; the ring never wraps inside a band
//    (its first two rows exist twice); where the ring is longer than the 16-bit offset field (fp16) the one register set is
//    moved by a constant between the bands that cross the middle -- 21 vector adds per band, outside the MFMA stream.
//  * Direct loads: a row is 8 (fp16) / 4 (int8) wave-wide loads of 16 pixels of one plane; a wave always fetches the same
//    planes and pixel halves, so its lanes' column terms are fixed registers.
#pragma once

#include "conv_patch.hpp"

namespace ckx {

// FUSED: fp16 -- bias + ReLU (EPI_ADD_RELU)
template <int DT, bool FUSED, int NW_ = 4, int AHEAD_ = 2>
struct ConvPatchWide
{
    static constexpr int ES     = DT == DT_I8 ? 1 : 2;
    static constexpr int CIN = 128, KO = 128, Y = 3, X = 3, TAPS = 9;
    static constexpr int TH     = 4;                     // output rows per band
    static constexpr int WO     = 28, MTW = TH * WO / 16; // 7 M tiles per band, shared by all waves
    static constexpr int NW     = NW_, NT = NW * 64;      // 8 waves x 16 channels or 4 waves x 32
    static constexpr int CPW    = KO / NW, NBT = CPW / 16; // channels and 16-channel weight tiles per wave
    static constexpr int AHEAD  = AHEAD_;
    static constexpr int PXB    = CIN * ES;              // bytes per pixel (256 / 128)
    static constexpr int KSP    = PXB / 64;              // MFMA k-steps per tap = planes of a ring row (4 / 2)
    static constexpr int PITCH  = 32;                    // pixels per ring row (Wo + 2 <= 32)
    static constexpr int PLANE  = PITCH * 64;
    static constexpr int ROWB   = KSP * PLANE;           // bytes per ring row (8192 / 4096)
    static constexpr int NEED   = TH + Y - 1;
    static constexpr int PERIOD = (NEED + AHEAD * TH + TH - 1) / TH * TH;
    static constexpr int NPH    = PERIOD / TH;
    static constexpr int PHYS   = PERIOD + Y - 1;
    static constexpr int RING_BYTES = PHYS * ROWB;
    static constexpr int LUT    = DT == DT_I8 ? 256 : 0;
    static constexpr int LDS    = RING_BYTES + LUT;
    static constexpr int NS     = KSP * TAPS;            // k-steps of a band (36 / 18)
    // the read addresses are moved by SPLIT rows between the bands below and above the middle of the ring where its
    // length exceeds the offset field
    static constexpr bool MOVES = (PERIOD - TH + Y - 1) * ROWB + (KSP - 1) * PLANE >= 65536;
    static constexpr int SPLIT  = MOVES ? TH * ((NPH + 1) / 2) : PERIOD;
    // a row's wave-wide loads, and the waves that share a row's loads / take alternate rows
    static constexpr int UPR    = KSP * (PITCH / 16);    // loads per row (8 / 4)
    static constexpr int NGRP   = NW > UPR ? NW / UPR : 1; // wave groups taking rows in turn
    static constexpr int UPW    = UPR > NW ? UPR / NW : 1; // load units of a row per wave
    static_assert((NW == 4 || NW == 8) && TH % NGRP == 0 && (Y - 1) % NGRP == 0 && NGRP * UPR == NW * UPW, "rows dealt evenly to the waves");
    static_assert(DT == DT_F16 || DT == DT_I8, "fp16 or int8");
    static_assert(!FUSED || DT == DT_F16, "fused epilogue: fp16 bias + ReLU");
    static_assert(LDS <= 160 * 1024, "the ring fits the LDS");
    static_assert((SPLIT - TH + Y - 1) * ROWB + (KSP - 1) * PLANE < 65536 &&
                      (PERIOD - TH - SPLIT + Y - 1) * ROWB + (KSP - 1) * PLANE < 65536,
                  "fragment read offsets fit the 16-bit field");
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    __device__ static __forceinline__ uint32_t key(uint32_t c) { return (c & 1u) | ((c >> 1) & 2u); }

    // The fragments that do not fit the AccVGPRs (W_V) stay in VGPRs: four waves may use 240 of their 256 AccVGPRs; with
    // two waves per SIMD (NW = 8) the compiler grants a wave 128 VGPRs and 128 AccVGPRs.
    static constexpr int W_A_FRAGS = (NW == 8 ? 128 : 240) / 4;   // weight fragments kept in AccVGPRs
    __host__ __device__ static constexpr bool w_in_vgpr(int tap, int ks, int j) { return (tap * KSP + ks) * NBT + j >= W_A_FRAGS; }

    // acc (+)= w x a: the weights out of AccVGPRs (W_V: VGPRs), pixels and accumulator in VGPRs; FIRST: the accumulator
    // starts at zero (the literal 0 as the addend)
    template <bool FIRST, bool W_V>
    __device__ static __forceinline__ void mfma(acc_t& c, const i32x4& w, const i32x4& a)
    {
#define CKX_WIDE_MFMA(OP)                                                             \
    if constexpr(W_V && FIRST)                                                        \
        asm volatile(OP " %0, %1, %2, 0" : "=v"(c) : "v"(w), "v"(a));                 \
    else if constexpr(W_V)                                                            \
        asm volatile(OP " %0, %1, %2, %0" : "+v"(c) : "v"(w), "v"(a));                \
    else if constexpr(FIRST)                                                          \
        asm volatile(OP " %0, %1, %2, 0" : "=v"(c) : "a"(w), "v"(a));                 \
    else                                                                              \
        asm volatile(OP " %0, %1, %2, %0" : "+v"(c) : "a"(w), "v"(a));
        if constexpr(DT == DT_I8)
        {
            CKX_WIDE_MFMA("v_mfma_i32_16x16x64_i8")
        }
        else
        {
            CKX_WIDE_MFMA("v_mfma_f32_16x16x32_f16")
        }
#undef CKX_WIDE_MFMA
    }

    __device__ static __forceinline__ void run(const ConvPatchArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        const uint32_t ring_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;

        const __amdgpu_buffer_rsrc_t rsrc_in   = make_rsrc(p.in, p.in_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_wei  = make_rsrc(p.wei, p.wei_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_none = make_rsrc(p.in, 0);
        const __amdgpu_buffer_rsrc_t rsrc_out  = make_rsrc(p.out, p.out_bytes);

        if constexpr(DT == DT_I8)
        {
            if(p.epi == EPI_REQUANT_RND)
                requant_lut_fill(smem + RING_BYTES, p.scale_relu, (int)threadIdx.x, NT);
        }

        // ---- weights: fragment (tap, k-step, channel tile j) of this wave. MFMA row frow = 4 q + i of tile j is output channel
        // CPW w + 4 NBT q + 4 j + i, so the lane in 16-lane row fq ends with the 4 NBT consecutive channels from
        // CPW w + 4 NBT fq on. Each workgroup starts at another filter row (all of them read the same weights at the same time).
        i32x4 wreg[TAPS][KSP][NBT];
        auto load_weights = [&](auto y0_c) {
            static_for<Y>([&](auto yy_c) {
                constexpr int y = (decltype(y0_c)::value + decltype(yy_c)::value) % Y;
#pragma unroll
                for(int j = 0; j < NBT; ++j)
                {
                    const uint32_t ch = (uint32_t)(CPW * wave) + (uint32_t)(4 * NBT) * (frow >> 2) + 4u * j + (frow & 3u);
#pragma unroll
                    for(int x = 0; x < X; ++x)
#pragma unroll
                        for(int ks = 0; ks < KSP; ++ks)
                            wreg[y * X + x][ks][j] = __builtin_bit_cast(
                                i32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                           rsrc_wei, (ch * TAPS + (uint32_t)(y * X + x)) * PXB + (uint32_t)ks * 64u + fq * 16u, 0, 0));
                }
            });
        };

        // ---- per-lane constants of the band's M tiles (the same for every wave) -------------------
        uint32_t rd[MTW][X];  // LDS address of the lane's pixel of tile t, shifted by tap column x, ring row 0 (+ moves), plane 0
        uint32_t rout = 0;    // output rows of the lane's pixels within the band, two bits per tile
        // byte offset of the lane's outputs of tile 0 relative to the band (a band's output rows are contiguous: tile t is
        // 16 t pixels further on, which travels in the scalar offset)
        const uint32_t ooff0 = (frow * KO + (uint32_t)(CPW * wave) + (uint32_t)(4 * NBT) * fq) * ES;
#pragma unroll
        for(int t = 0; t < MTW; ++t)
        {
            const uint32_t q = (uint32_t)(t * 16) + frow;
            const uint32_t r = magic_div(q, p.div_wo);
            const uint32_t w = q - r * (uint32_t)p.Wo;
            rout |= r << (2 * t);
#pragma unroll
            for(int x = 0; x < X; ++x)
            {
                const uint32_t cc = w + (uint32_t)x;
                rd[t][x]          = ring_lds + r * ROWB + cc * 64u + ((fq ^ key(cc)) << 4);
            }
        }
        static_assert(TH <= 4, "two bits per tile row");
        float bias4[4 * NBT];
#pragma unroll
        for(int i = 0; i < 4 * NBT; ++i)
            bias4[i] = FUSED ? (float)reinterpret_cast<const _Float16*>(p.bias)[CPW * wave + 4 * NBT * (int)fq + i] : 0.0f;

        // ---- input rows -> ring. Wave w fetches load unit w % UPR (plane unit / 2, pixels 16 (unit % 2) .. + 15) of the rows
        // i = w / UPR, w / UPR + NGRP, ... : lane -> pixel 16 (unit % 2) + lane / 4, LDS chunk position lane % 4 <- global chunk
        // 4 plane + (position ^ key(pixel)). The row travels in the scalar offset; a row outside the image is fetched
        // through a buffer resource of zero bytes (zero fill).
        const int grp = wave / UPR; // (NW <= UPR: 0)
        uint32_t gcol[UPW];
        uint32_t dst_off[UPW];      // LDS offset of the wave's load units within a ring row
#pragma unroll
        for(int u = 0; u < UPW; ++u)
        {
            const int unit = wave % UPR + NW * u; // (UPW > 1: the wave takes units w, w + NW, ...)
            const int cc = 16 * (unit % 2) + lane / 4, wi = cc - p.pL;
            gcol[u]    = (uint32_t)wi < (uint32_t)p.Wi ? (uint32_t)wi * PXB + (uint32_t)(unit / 2) * 64u + ((((uint32_t)lane & 3u) ^ key((uint32_t)cc)) << 4)
                                                       : kOutOfRange;
            dst_off[u] = (uint32_t)((unit / 2) * PLANE + (unit % 2) * 1024);
        }
        // patch row j of image n (input row j - pT) into physical ring row slot: the wave's UPW load units of it
        auto load_row = [&](int n, int j, int slot) {
            const int hi        = j - p.pT;
            const bool ok       = (uint32_t)hi < (uint32_t)p.Hi;
            const uint32_t soff = (uint32_t)((n * p.Hi + (ok ? hi : 0)) * p.Wi) * PXB;
#pragma unroll
            for(int u = 0; u < UPW; ++u)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(ok ? rsrc_in : rsrc_none,
                                                         (lds_ptr_t)(smem + __builtin_amdgcn_readfirstlane(dst_off[u]) + slot * ROWB), 16,
                                                         gcol[u], soff, 0, 0);
        };

        acc_t acc[MTW][NBT];
        // pixel fragments: a ring of NF register tuples over the band's NS * MTW (k-step, tile) pairs in order; the fragment NF
        // pairs ahead is requested into the tuple an MFMA has just read
        constexpr int NF = NW == 4 ? 7 : (DT == DT_I8 ? 5 : 3), NPAIR = NS * MTW; // (eight fp16 waves: what their 128 VGPRs leave room for)
        i32x4 af[NF];

        // fragment of M tile T for k-step S of the band at ring position PH (the registers stand SPLIT rows further on
        // for the bands above the middle)
        auto read_pair = [&](auto ph_c, auto k_c) {
            constexpr int PH = decltype(ph_c)::value, K = decltype(k_c)::value, S = K / MTW, T = K % MTW;
            constexpr int tap = S / KSP, ks = S % KSP, y = tap / X, x = tap % X;
            af[K % NF] = lds_read_b128<((PH < SPLIT ? PH : PH - SPLIT) + y) * ROWB + ks * PLANE>(rd[T][x]);
        };
        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        const int nbands = (p.Ho + TH - 1) / TH;

        // ---- epilogue of M tile T of band bd: four consecutive channels of one pixel per lane, through a buffer
        // resource (a pixel row past Ho gets the out-of-range offset and is dropped)
        auto store_tile = [&](auto t_c, auto epi_c, int n, int bd) {
            constexpr int t = decltype(t_c)::value, EPI = decltype(epi_c)::value;
            const uint32_t soff = (uint32_t)((n * p.Ho + TH * bd) * p.Wo + 16 * t) * (KO * ES);
            const uint32_t voff = (int)((rout >> (2 * t)) & 3u) < p.Ho - TH * bd ? ooff0 : kOutOfRange;
            if constexpr(DT == DT_I8)
            {
                int o[NBT];
                if constexpr(EPI == EPI_REQUANT_RND)
                {
                    i32x4 vv[NBT];
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        vv[j] = acc[t][j];
                    int bb[4 * NBT];
                    requant_lut<NBT>(vv, p.scale_gemm, ring_lds + (uint32_t)RING_BYTES, bb);
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        o[j] = pack4_low_bytes(bb[4 * j], bb[4 * j + 1], bb[4 * j + 2], bb[4 * j + 3]);
                }
                else
                {
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        o[j] = pack4_low_bytes(epilogue_i8<EPI>(acc[t][j][0], p.scale_gemm, p.scale_relu), epilogue_i8<EPI>(acc[t][j][1], p.scale_gemm, p.scale_relu),
                                               epilogue_i8<EPI>(acc[t][j][2], p.scale_gemm, p.scale_relu), epilogue_i8<EPI>(acc[t][j][3], p.scale_gemm, p.scale_relu));
                }
                if constexpr(NBT == 2)
                    __builtin_amdgcn_raw_buffer_store_b64(i32x2{o[0], o[NBT - 1]}, rsrc_out, voff, soff, 0);
                else
                    __builtin_amdgcn_raw_buffer_store_b32(o[0], rsrc_out, voff, soff, 0);
            }
            else
            {
                typedef _Float16 f16xn __attribute__((ext_vector_type(4 * NBT)));
                f16xn o;
#pragma unroll
                for(int j = 0; j < NBT; ++j)
#pragma unroll
                    for(int i = 0; i < 4; ++i)
                    {
                        float x = acc[t][j][i];
                        if constexpr(EPI == EPI_ADD_RELU)
                            x = __builtin_fmaxf(x + bias4[4 * j + i], 0.0f);
                        o[4 * j + i] = (_Float16)x;
                    }
                if constexpr(NBT == 2)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, o), rsrc_out, voff, soff, 0);
                else
                    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(i32x2, o), rsrc_out, voff, soff, 0);
            }
        };

        // One band (index b of image n) at ring position PH. Returns after the band's stores have been issued, with the
        // first fragments of the next band (if there is one) on their way.
        auto band = [&](auto ph_c, auto epi_c, int n, int b) {
            constexpr int PH  = decltype(ph_c)::value;
            constexpr int PHN = (PH + TH) % PERIOD;
            // the TH new rows of band b + AHEAD go to logical rows (PH + AHEAD * TH + Y - 1 + i) % PERIOD; those that land
            // on the first Y - 1 rows are also loaded behind the end
            constexpr int L0   = (PH + AHEAD * TH + Y - 1) % PERIOD;
            constexpr bool DUP = L0 + TH > PERIOD;
            constexpr int NLW  = (TH + (DUP ? Y - 1 : 0)) / NGRP;       // loads of this wave in this band
            const int jnew     = TH * (b + AHEAD) + Y - 1;              // first new patch row

            static_for<NS>([&](auto s_c) {
                constexpr int s = decltype(s_c)::value;
                static_for<MTW>([&](auto g_c) {
                    constexpr int g = decltype(g_c)::value;
                    // This pair's fragment has landed: LDS reads return in order, and behind it the wave has issued the
                    // fragments of the next NF - 1 pairs (fewer at the band's end).
                    constexpr int k = s * MTW + g;
                    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(k + NF <= NPAIR ? NF - 1 : NPAIR - 1 - k) : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<NBT>([&](auto j_c) {
                        constexpr int j = decltype(j_c)::value;
                        mfma<s == 0, w_in_vgpr(s / KSP, s % KSP, j)>(acc[g][j], wreg[s / KSP][s % KSP][j], af[k % NF]);
                    });
                    if constexpr(k + NF < NPAIR)
                        read_pair(ph_c, std::integral_constant<int, k + NF>{});
                    // direct loads of this wave's rows of band b + AHEAD, over the first five eighths of the band
                    constexpr int idx = s * MTW + g, SPAN = NS * MTW * 5 / 8;
                    constexpr int li  = idx * NLW / SPAN;
                    if constexpr(li < NLW && (idx == 0 || (idx - 1) * NLW / SPAN < li))
                    {
                        // the li-th row of this wave: new row i = grp + NGRP li (< TH), or the copy of new row PERIOD - L0 + ...
                        const int i = grp + NGRP * li;
                        if constexpr(li < TH / NGRP)
                        {
                            int slot = L0 + i;
                            slot     = slot >= PERIOD ? slot - PERIOD : slot;
                            load_row(n, jnew + i, slot);
                        }
                        else
                        {
                            const int d = grp + NGRP * (li - TH / NGRP);   // 0 .. Y - 2
                            load_row(n, jnew + (PERIOD - L0) + d, PERIOD + d);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });

            // the next band's rows have landed (this wave's share): a wave's loads retire in order, the stores of the band
            // before are older still, and what may remain are the loads issued in this band body (AHEAD = 2)
            static_assert(AHEAD == 1 || AHEAD == 2, "the wait below counts this band's loads only");
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * NLW * UPW) : "memory");
            barrier();
            if constexpr(MOVES && (PHN == SPLIT || PHN == 0))
            {
                // the next band reads on the other side of the middle of the ring
#pragma unroll
                for(int t = 0; t < MTW; ++t)
#pragma unroll
                    for(int x = 0; x < X; ++x)
                        rd[t][x] += PHN == SPLIT ? (uint32_t)(SPLIT * ROWB) : (uint32_t)(-(SPLIT * ROWB));
            }
            if(b + 1 < nbands)
                static_for<NF>([&](auto k_c) { read_pair(std::integral_constant<int, PHN>{}, k_c); });
            // (the MFMA results must have left the pipeline before the epilogue reads them: inline-assembly MFMAs are
            // invisible to the compiler's hazard handling)
            asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            static_for<MTW>([&](auto t_c) { store_tile(t_c, epi_c, n, b); });
        };

        // rows of the first band and of the AHEAD - 1 bands after it: this wave's share
        constexpr int NFIRST = (NEED + TH * (AHEAD - 1)) / NGRP;
        static_assert((NEED + TH * (AHEAD - 1)) % NGRP == 0, "first rows dealt evenly");
        auto first_rows = [&](int n) {
#pragma unroll
            for(int k = 0; k < NFIRST; ++k)
                load_row(n, grp + NGRP * k, grp + NGRP * k);
        };
        auto image = [&](auto epi_c, int n, bool first) {
            // Only the first band's rows have to land before the MFMAs start: a wave's loads retire in order, and behind them
            // are the later bands' rows and, in the first image, the weights
            if(first)
            {
                // (the counter holds 63: with more loads behind, a few of the weights are waited for as well)
                constexpr int behind = (AHEAD - 1) * TH / NGRP * UPW + TAPS * KSP * NBT;
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(behind < 63 ? behind : 63) : "memory");
            }
            else
            {
                first_rows(n);
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * TH / NGRP * UPW) : "memory");
            }
            barrier();
            static_for<NF>([&](auto k_c) { read_pair(std::integral_constant<int, 0>{}, k_c); });
            // the band loop, unrolled over the ring's period
            int b = 0;
            for(;;)
            {
                bool done = false;
                static_for<NPH>([&](auto k_c) {
                    if(!done)
                    {
                        band(std::integral_constant<int, decltype(k_c)::value * TH>{}, epi_c, n, b);
                        done = ++b == nbands;
                    }
                });
                if(done)
                    break;
            }
            // the read addresses back at the start of the ring for the next image (b bands from position 0)
            if constexpr(MOVES)
            {
                if(((nbands % NPH) * TH) >= SPLIT)
                {
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
#pragma unroll
                        for(int x = 0; x < X; ++x)
                            rd[t][x] -= (uint32_t)(SPLIT * ROWB);
                }
            }
            barrier(); // the ring is free for the next image's first rows
        };
        using std::integral_constant;
        first_rows((int)blockIdx.x);
        switch(blockIdx.x % 3)
        {
        case 0: load_weights(integral_constant<int, 0>{}); break;
        case 1: load_weights(integral_constant<int, 1>{}); break;
        default: load_weights(integral_constant<int, 2>{}); break;
        }
        bool first = true;
        for(int n = (int)blockIdx.x; n < p.N; n += (int)gridDim.x, first = false)
        {
            if constexpr(DT == DT_I8)
            {
                if(p.epi == EPI_REQUANT_RND)
                    image(integral_constant<int, EPI_REQUANT_RND>{}, n, first);
                else if(p.epi == EPI_REQUANT_CK)
                    image(integral_constant<int, EPI_REQUANT_CK>{}, n, first);
                else
                    image(integral_constant<int, EPI_PASSTHROUGH>{}, n, first);
            }
            else if constexpr(FUSED)
                image(integral_constant<int, EPI_ADD_RELU>{}, n, first);
            else
                image(integral_constant<int, EPI_PASSTHROUGH>{}, n, first);
        }
        // loads of rows past the last band still target this workgroup's LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
};

template <int DT, bool FUSED>
__global__ __launch_bounds__((ConvPatchWide<DT, FUSED>::NT)) void conv_patch_wide_kernel(const ConvPatchArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_patch_smem[];
    ConvPatchWide<DT, FUSED>::run(p, ckx_patch_smem);
}

// (conv_patch.hip) dt: DT_F16 / DT_I8; fused: bias + ReLU (fp16); C = K = 128, Wo = 28
hipError_t launch_conv_patch_wide(int dt, bool fused, const ConvPatchArgs& a, hipStream_t s);

} // namespace ckx
