// Input-patch conv2d forward for gfx950, fp16 and int8, NHWC / KYXC / NHWK: 3 x 3 layers with 64 input and 64 output
// channels (ResNet conv2_x, 56 x 56), where the implicit-GEMM tile kernel re-reads every input pixel once per filter tap
// out of L2 and is bound by that.
//
// Takes the place of the same reference kernel as the tile kernel
// (DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K,
// device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720) for the shapes it covers:
//   C = 64, K = 64, 3 x 3 taps, stride 1, dilation 1, Wo = 8 * MTW <= 56 (Wo + 2 <= 64).
//
//  * A workgroup (4 waves, one per SIMD) owns whole images and walks them in bands of TH output rows. The input rows of
//    a band (TH + 2) live in LDS in a ring of rows; the rows of the band(s) after it are fetched by direct global->LDS
//    loads while the band is multiplied. Every input pixel is read from memory once.
//  * THE WEIGHTS LIVE IN REGISTERS: a wave keeps the 9 taps x 64 input channels of its output channels as 36 MFMA
//    operand fragments in 144 AccVGPRs for the life of the workgroup (an MFMA takes either operand from either
//    register file), next to its accumulators. No weight ever passes through LDS, and the LDS is the ring's alone.
//  * NOTHING BUT MFMAs AND FRAGMENT READS IN THE BAND LOOP. With one wave per SIMD a vector-ALU instruction between two
//    MFMAs costs about seven cycles of the matrix pipeline, so the address of every fragment read is a per-lane register
//    that never changes plus a compile-time offset:
//      - a ring row is two planes of 64 pixels x 64 bytes (fp16: channels 0..31 / 32..63 = the two MFMA k-steps of a
//        tap; int8: one plane), so the k-step is an offset; 16-byte chunks are swizzled inside a 64-byte pixel by bits
//        0 and 2 of the pixel column (conflict free under the LDS' lane grouping);
//      - the tap column x selects one of three per-lane registers (the swizzle depends on the column);
//      - the tap row y and the band's position in the ring are offsets: the band loop is unrolled over the ring's
//        period, and the ring never wraps inside a band -- its first two rows exist twice, once at the start and once
//        behind the end, and the input rows that land there are loaded into both places.
//  * D^T = B_frag x A_frag with the weight rows dealt to the MFMA rows so that a lane ends up with 8 (fp16) or 16 (int8)
//    consecutive channels of one pixel: one 16-byte store, no trip through LDS.
//  * fp16 (plain epilogue): a band's conversions and stores run INSIDE the next band's MFMA stream (two accumulator sets,
//    one M tile every second k-step), so the matrix pipeline does not idle during an epilogue and the stores leave spread
//    over the band instead of in a burst.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct ConvPatchArgs
{
    const void* in;
    const void* wei;
    void* out;
    uint32_t in_bytes, wei_bytes, out_bytes; // (out_bytes: also the extent of the residual tensor)
    int N, Hi, Wi, Ho, Wo;
    int pT, pL;
    MagicDiv div_wo;
    int epi; // fp16: EPI_PASSTHROUGH, EPI_ADD_RELU, EPI_ADD_RELU_ADD; int8: EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND,
             // EPI_MUL2_CLAMP / EPI_RELU_MUL2_CLAMP (one requant scale per output channel)
    const void* bias; // [64]: fp16 bias (fp16 kernels), fp32 requant scales (the int8 per-channel variant)
    const void* resi; // NHWK fp16
    float scale_gemm, scale_relu; // int8 requant epilogues
};

// FUSED: fp16 -- the add / ReLU epilogues (bias, residual); int8 -- one requant scale per output channel
// fp16: bands of 4 rows, 2 x 2 waves (a wave: 16 * MTW pixels x 32 channels); int8: bands of 8 rows, 4 x 1 waves (a wave:
// 16 * MTW pixels x all 64 channels). Either way a wave holds 36 weight fragments and MTW * NBT accumulator tiles.
template <int DT, int MTW, bool FUSED, bool PIPE_ = (DT == DT_F16 && !FUSED), int AHEAD_ = 2>
struct ConvPatch
{
    static constexpr int ES     = DT == DT_I8 ? 1 : 2;
    static constexpr int TH     = DT == DT_I8 ? 8 : 4;   // output rows per band
    static constexpr int WMW    = DT == DT_I8 ? 4 : 2;   // waves along the pixels
    static constexpr int WNW    = 4 / WMW;               // waves along the output channels
    static constexpr int NBT    = 4 / WNW;               // 16-channel weight tiles per wave (2 / 4)
    static constexpr int CPW    = 16 * NBT;              // channels per wave
    static constexpr int Y = 3, X = 3, TAPS = 9, KO = 64;
    static constexpr bool PIPE  = PIPE_;                 // the epilogue of a band runs inside the next band's MFMA stream
    static constexpr int AHEAD  = AHEAD_;                // bands of input rows in flight ahead of the band being multiplied
    static constexpr int PXB    = 64 * ES;               // bytes per pixel
    static constexpr int KSP    = PXB / 64;              // MFMA k-steps per tap = planes of a ring row (2 / 1)
    static constexpr int PLANE  = 64 * 64;               // 64 pixels x 64 bytes
    static constexpr int ROWB   = KSP * PLANE;           // bytes per ring row
    static constexpr int NEED   = TH + Y - 1;            // input rows of one band
    static constexpr int PERIOD = (NEED + AHEAD * TH + TH - 1) / TH * TH; // logical ring rows, a multiple of TH
    static constexpr int NPH    = PERIOD / TH;           // band positions in the ring = copies of the band body
    static constexpr int PHYS   = PERIOD + Y - 1;        // physical rows: the first Y - 1 once more behind the end
    static constexpr int RING_BYTES = PHYS * ROWB;
    static constexpr int LUT    = DT == DT_I8 ? 256 : 0; // table of the rounded requant epilogue
    static constexpr int LDS    = RING_BYTES + LUT;
    static constexpr int NT     = 256;
    static constexpr int NS     = KSP * TAPS;            // k-steps of a band
    // a lane's read addresses come in two sets, the second SPLIT rows further on: the offset field has 16 bits
    static constexpr int SPLIT  = TH * ((NPH + 1) / 2);
    // (Every accumulator lives in VGPRs, which the register-resident weights leave free: results in AccVGPRs cost a read
    // instruction per value in the epilogue -- int8 33.5 -> 31.7 us at N = 256 without them; fp16 level.)
    static_assert(MTW >= 1 && MTW <= 7, "covered widths");
    static_assert(DT == DT_F16 || DT == DT_I8, "fp16 or int8");
    static_assert(LDS <= 160 * 1024, "the ring fits the LDS");
    static_assert((SPLIT - TH + Y - 1) * ROWB + (KSP - 1) * PLANE < 65536 &&
                      (PERIOD - TH - SPLIT + Y - 1) * ROWB + (KSP - 1) * PLANE < 65536,
                  "fragment read offsets fit the 16-bit field");
    static constexpr bool F16FUSED = FUSED && DT == DT_F16, I8PERCH = FUSED && DT == DT_I8;
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    // swizzle key of a pixel column: the 16 pixels of a fragment read must land on distinct banks (a ds_read_b128 is
    // served in four cycles; the 16 lanes of a cycle are those with equal (lane bit 5, parity of lane bits 2..4))
    __device__ static __forceinline__ uint32_t key(uint32_t c) { return (c & 1u) | ((c >> 1) & 2u); }

    // acc (+)= w x a: the weights out of AccVGPRs, pixels and accumulator in VGPRs. Inline assembly: the operand
    // constraints are what places the weights in the AccVGPR half of the register file. FIRST: the accumulator starts at
    // zero (the literal 0 as the addend), which saves zeroing it for every band.
    template <bool FIRST>
    __device__ static __forceinline__ void mfma(acc_t& c, const i32x4& w, const i32x4& a)
    {
        if constexpr(DT == DT_I8 && FIRST)
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, 0" : "=v"(c) : "a"(w), "v"(a));
        else if constexpr(DT == DT_I8)
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(c) : "a"(w), "v"(a));
        else if constexpr(FIRST)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=v"(c) : "a"(w), "v"(a));
        else
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "a"(w), "v"(a));
    }

    __device__ static __forceinline__ void run(const ConvPatchArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int wm = wave / WNW, wn = wave % WNW;
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        const uint32_t ring_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;

        const __amdgpu_buffer_rsrc_t rsrc_in  = make_rsrc(p.in, p.in_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_wei = make_rsrc(p.wei, p.wei_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_none = make_rsrc(p.in, 0);
        const __amdgpu_buffer_rsrc_t rsrc_out  = make_rsrc(p.out, p.out_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_resi = make_rsrc(p.resi ? p.resi : p.out, p.resi ? p.out_bytes : 0);

        if constexpr(DT == DT_I8)
        {
            if(p.epi == EPI_REQUANT_RND)
                requant_lut_fill(smem + RING_BYTES, p.scale_relu, (int)threadIdx.x, 256);
        }

        // ---- weights: fragment (tap, k-step, channel tile j) of this wave. MFMA row frow = 4 * q + i of tile j is output
        // channel CPW * wn + 4 * NBT * q + 4 * j + i, so that the lane in 16-lane row fq ends with the 4 * NBT
        // consecutive channels from CPW * wn + 4 * NBT * fq on.
        // All workgroups read the same 72 KB at the same time: each starts at another filter row, so that the L2 lines in
        // demand at any moment are three times as many.
        i32x4 wreg[TAPS][KSP][NBT];
        auto load_weights = [&](auto y0_c) {
            static_for<Y>([&](auto yy_c) {
                constexpr int y = (decltype(y0_c)::value + decltype(yy_c)::value) % Y;
#pragma unroll
                for(int j = 0; j < NBT; ++j)
                {
                    const uint32_t ch = (uint32_t)(CPW * wn) + (uint32_t)(4 * NBT) * (frow >> 2) + 4u * j + (frow & 3u);
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

        // ---- per-lane constants of the wave's M tiles -----------------------------------
        uint32_t rd0[MTW][X]; // LDS address of the lane's pixel of tile t, shifted by tap column x, in ring row 0, plane 0
        uint32_t rd1[MTW][X]; // ... SPLIT rows further on
        uint32_t rout[MTW];   // output row of the lane's pixel within the band
        uint32_t ooff[MTW];   // byte offset of the lane's outputs relative to the band
#pragma unroll
        for(int t = 0; t < MTW; ++t)
        {
            const uint32_t q = (uint32_t)((wm * MTW + t) * 16) + frow;
            const uint32_t r = magic_div(q, p.div_wo);
            const uint32_t w = q - r * (uint32_t)p.Wo;
            rout[t]          = r;
            ooff[t]          = ((r * (uint32_t)p.Wo + w) * KO + (uint32_t)(CPW * wn) + (uint32_t)(4 * NBT) * fq) * ES;
#pragma unroll
            for(int x = 0; x < X; ++x)
            {
                const uint32_t cc = w + (uint32_t)x;
                rd0[t][x]         = ring_lds + r * ROWB + cc * 64u + ((fq ^ key(cc)) << 4);
                rd1[t][x]         = rd0[t][x] + (uint32_t)(SPLIT * ROWB);
            }
        }
        // fused add / ReLU epilogues: the lane's 8 bias values once, its residual values band by band
        const bool has_resi = F16FUSED && p.epi == EPI_ADD_RELU_ADD;
        f16x8 bias8 = {0, 0, 0, 0, 0, 0, 0, 0};
        if constexpr(F16FUSED)
            bias8 = *reinterpret_cast<const f16x8*>(reinterpret_cast<const _Float16*>(p.bias) + CPW * wn + 4 * NBT * (int)fq);
        f16x8 resi8[F16FUSED ? MTW : 1];
#pragma unroll
        for(int t = 0; t < (F16FUSED ? MTW : 1); ++t)
            resi8[t] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        // int8, per-channel requant: the scales of the lane's 16 consecutive channels, for the life of the workgroup
        float chsc[I8PERCH ? 4 * NBT : 1];
        if constexpr(I8PERCH)
        {
#pragma unroll
            for(int e = 0; e < 4 * NBT; ++e)
                chsc[e] = reinterpret_cast<const float*>(p.bias)[CPW * wn + 4 * NBT * (int)fq + e];
        }

        // ---- input rows -> ring. A wave-wide direct load fills 16 pixels of one plane; wave w always fetches pixels
        // 16 w .. 16 w + 15 of a row (both planes), so its lanes' column terms are fixed: lane -> pixel 16 w + lane / 4,
        // LDS chunk position lane % 4 <- global chunk 4 * plane + (position ^ key(pixel)). The row travels in the
        // scalar offset; a row outside the image is fetched through a buffer resource of zero bytes (every lane out of range:
        // zero fill), which costs a scalar select where a per-lane offset would cost a vector instruction.
        uint32_t gcol[KSP];
        {
            const int cc = 16 * wave + lane / 4, wi = cc - p.pL;
#pragma unroll
            for(int h = 0; h < KSP; ++h)
                gcol[h] = (uint32_t)wi < (uint32_t)p.Wi
                              ? (uint32_t)wi * PXB + (uint32_t)h * 64u + ((((uint32_t)lane & 3u) ^ key((uint32_t)cc)) << 4)
                              : kOutOfRange;
        }
        uint8_t* wave_dst = smem + wave * 1024;
        // patch row j of image n (input row j - pT), plane h, into physical ring row SLOT
        auto load_row = [&](int n, int j, auto slot_c, auto h_c) {
            constexpr int SLOT = decltype(slot_c)::value, H = decltype(h_c)::value;
            const int hi        = j - p.pT;
            const bool ok       = (uint32_t)hi < (uint32_t)p.Hi;
            const uint32_t soff = (uint32_t)((n * p.Hi + (ok ? hi : 0)) * p.Wi) * PXB;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ok ? rsrc_in : rsrc_none, (lds_ptr_t)(wave_dst + SLOT * ROWB + H * PLANE), 16,
                                                     gcol[H], soff, 0, 0);
        };

        // two accumulator sets: a band is multiplied into one while the band before it leaves the other. Without PIPE only
        // set 0 exists.
        acc_t acc0[MTW][NBT], acc1[PIPE ? MTW : 1][NBT];
        i32x4 af[2][MTW];

        // fragment of M tile T for k-step S of the band at ring position PH
        auto read_one = [&](auto ph_c, auto s_c, auto t_c) {
            constexpr int PH = decltype(ph_c)::value, S = decltype(s_c)::value, T = decltype(t_c)::value;
            constexpr int tap = S / KSP, ks = S % KSP, y = tap / X, x = tap % X;
            if constexpr(PH < SPLIT)
                af[S & 1][T] = lds_read_b128<(PH + y) * ROWB + ks * PLANE>(rd0[T][x]);
            else
                af[S & 1][T] = lds_read_b128<(PH - SPLIT + y) * ROWB + ks * PLANE>(rd1[T][x]);
        };
        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };
        const int nbands = (p.Ho + TH - 1) / TH;

        // (The variant with the residual input moves three tensors: its output, from 64 MiB on, is stored non-temporally --
        // measured 72 -> 67 us at N = 256, where the plain fp16 kernel loses 2 us with such stores.)
        const bool nt_out = F16FUSED && p.out_bytes >= (64u << 20);
        auto store_out    = [&](i32x4 x, uint32_t voff, uint32_t soff) {
            if(nt_out)
                __builtin_amdgcn_raw_buffer_store_b128(x, rsrc_out, voff, soff, 2);
            else
                __builtin_amdgcn_raw_buffer_store_b128(x, rsrc_out, voff, soff, 0);
        };
        // ---- epilogue of M tile T of band bd out of accumulator set SET: 4 * NBT consecutive channels of one pixel per lane.
        // The store goes through a buffer resource: a pixel row past Ho (the last band's, or a band that does not exist)
        // gets the out-of-range offset and is dropped, so the code carries no branch. EPI: the functor as a compile-time
        // constant (tested per value it would turn into hundreds of scalar branches).
        auto store_tile = [&](auto set_c, auto t_c, auto epi_c, int n, int bd) {
            constexpr int SET = decltype(set_c)::value, t = decltype(t_c)::value, EPI = decltype(epi_c)::value;
            acc_t v[NBT];
#pragma unroll
            for(int j = 0; j < NBT; ++j)
                v[j] = SET == 1 ? acc1[PIPE ? t : 0][j] : acc0[t][j];
            const uint32_t soff = (uint32_t)((n * p.Ho + TH * (bd < 0 ? 0 : bd)) * p.Wo) * (KO * ES);
            const uint32_t voff = (int)rout[t] < (bd < 0 ? 0 : p.Ho - TH * bd) ? ooff[t] : kOutOfRange;
            if constexpr(DT == DT_I8)
            {
                int o[NBT];
                if constexpr(EPI == EPI_MUL2_CLAMP || EPI == EPI_RELU_MUL2_CLAMP)
                {
                    constexpr bool relu = EPI == EPI_RELU_MUL2_CLAMP;
                    constexpr int NSC   = I8PERCH ? 4 * NBT : 1;
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        o[j] = pack4_low_bytes(mul2_clamp(v[j][0], chsc[(4 * j) % NSC], relu), mul2_clamp(v[j][1], chsc[(4 * j + 1) % NSC], relu),
                                               mul2_clamp(v[j][2], chsc[(4 * j + 2) % NSC], relu), mul2_clamp(v[j][3], chsc[(4 * j + 3) % NSC], relu));
                }
                else if constexpr(EPI == EPI_REQUANT_RND)
                {
                    int bb[4 * NBT];
                    requant_lut<NBT>(v, p.scale_gemm, ring_lds + (uint32_t)RING_BYTES, bb);
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        o[j] = pack4_low_bytes(bb[4 * j], bb[4 * j + 1], bb[4 * j + 2], bb[4 * j + 3]);
                }
                else
                {
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                        o[j] = pack4_low_bytes(epilogue_i8<EPI>(v[j][0], p.scale_gemm, p.scale_relu), epilogue_i8<EPI>(v[j][1], p.scale_gemm, p.scale_relu),
                                               epilogue_i8<EPI>(v[j][2], p.scale_gemm, p.scale_relu), epilogue_i8<EPI>(v[j][3], p.scale_gemm, p.scale_relu));
                }
                store_out(i32x4{o[0], o[1], o[2], o[3]}, voff, soff);
            }
            else
            {
                f16x8 o;
#pragma unroll
                for(int i = 0; i < 4; ++i)
                {
                    float v0 = v[0][i], v1 = v[1][i];
                    if constexpr(EPI != EPI_PASSTHROUGH)
                    {
                        v0 = epi_f16_value(EPI, v0, (float)bias8[i], (float)resi8[F16FUSED ? t : 0][i]);
                        v1 = epi_f16_value(EPI, v1, (float)bias8[4 + i], (float)resi8[F16FUSED ? t : 0][4 + i]);
                    }
                    o[i]     = (_Float16)v0;
                    o[4 + i] = (_Float16)v1;
                }
                store_out(__builtin_bit_cast(i32x4, o), voff, soff);
            }
        };
        // residual values of band bd (the add / ReLU / add epilogue): plain loads through a buffer resource, rows past Ho
        // read as zero
        auto load_resi = [&](int n, int bd) {
            if constexpr(F16FUSED)
                if(has_resi)
                {
                    const uint32_t soff = (uint32_t)((n * p.Ho + TH * (bd < 0 ? 0 : bd)) * p.Wo) * (KO * ES);
                    const int rows      = bd < 0 ? 0 : p.Ho - TH * bd;
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
                        resi8[F16FUSED ? t : 0] = __builtin_bit_cast(
                            f16x8, __builtin_amdgcn_raw_buffer_load_b128(rsrc_resi, (int)rout[t] < rows ? ooff[t] : kOutOfRange, soff, 0));
                }
        };

        // One band (index b of image n) at ring position PH, multiplied into accumulator set SET. PIPE: the band before it
        // (b - 1, or none: then every store is out of range) leaves the other set meanwhile, one M tile per DRAIN_EVERY
        // k-steps, so that its conversions and stores run in the shadow of this band's MFMAs. Returns with the first
        // fragments of the next band (if there is one) on their way.
        auto band = [&](auto ph_c, auto set_c, auto epi_c, int n, int b) {
            constexpr int PH = decltype(ph_c)::value, SET = decltype(set_c)::value;
            constexpr int PHN = (PH + TH) % PERIOD;                  // ring position of the next band
            // the TH new rows of band b + AHEAD go to logical rows (PH + AHEAD * TH + Y - 1 + i) % PERIOD; those that
            // land on the first Y - 1 rows are also loaded behind the end
            constexpr int L0   = (PH + AHEAD * TH + Y - 1) % PERIOD;
            constexpr bool DUP = L0 + TH > PERIOD;
            constexpr int NROW = TH + (DUP ? Y - 1 : 0), NL = NROW * KSP; // loads of this wave in this band
            constexpr int DRAIN_EVERY = (NS - 2) / MTW;                  // fp16: 2, int8: 1
            static_assert(!PIPE || DRAIN_EVERY >= 1, "one k-step per drained tile");
            const int jnew     = TH * (b + AHEAD) + Y - 1;               // first new patch row

            // residual values of the band whose epilogue runs in this body: before the band's direct loads
            load_resi(n, PIPE ? b - 1 : b);

            static_for<NS>([&](auto s_c) {
                constexpr int s = decltype(s_c)::value;
                static_for<MTW>([&](auto g_c) {
                    constexpr int g = decltype(g_c)::value;
                    // This tile's fragment has landed. LDS reads return in order, and behind it the wave has issued the
                    // fragments of the tiles after it and, for the next k-step, those of the tiles before it: MTW - 1 reads.
                    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(s + 1 < NS ? MTW - 1 : MTW - 1 - g) : "memory");
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<NBT>([&](auto j_c) {
                        constexpr int j = decltype(j_c)::value;
                        {
                            if constexpr(SET == 1)
                                mfma<s == 0>(acc1[PIPE ? g : 0][j], wreg[s / KSP][s % KSP][j], af[s & 1][g]);
                            else
                                mfma<s == 0>(acc0[g][j], wreg[s / KSP][s % KSP][j], af[s & 1][g]);
                        }
                        // the same tile's fragment of the next k-step, behind the tile's first MFMA: a whole k-step to land
                        if constexpr(j == 0 && s + 1 < NS)
                            read_one(ph_c, std::integral_constant<int, s + 1>{}, g_c);
                    });
                    // direct loads of the rows of band b + AHEAD: NL of them over the first five eighths of the band
                    constexpr int idx = s * MTW + g, SPAN = NS * MTW * 5 / 8;
                    constexpr int li  = idx * NL / SPAN;
                    if constexpr(li < NL && (idx == 0 || (idx - 1) * NL / SPAN < li))
                    {
                        constexpr int i = li / KSP, h = li % KSP;   // row i of the new rows (TH .. : the copies), plane h
                        if constexpr(i < TH)
                            load_row(n, jnew + i, std::integral_constant<int, (L0 + i) % PERIOD>{}, std::integral_constant<int, h>{});
                        else
                            load_row(n, jnew + (PERIOD - L0) + (i - TH), std::integral_constant<int, PERIOD + (i - TH)>{},
                                     std::integral_constant<int, h>{});
                    }
                    // the band before this one: M tile (s - 1) / DRAIN_EVERY behind the tile in the middle of the k-step
                    constexpr int td = s >= 1 && (s - 1) / DRAIN_EVERY < MTW ? (s - 1) / DRAIN_EVERY : 0;
                    if constexpr(PIPE && g == MTW / 2 && s >= 1 && (s - 1) % DRAIN_EVERY == 0 && (s - 1) / DRAIN_EVERY < MTW)
                        store_tile(std::integral_constant<int, 1 - SET>{}, std::integral_constant<int, td>{}, epi_c, n, b - 1);
                    __builtin_amdgcn_sched_barrier(0);
                });
            });

            // The next band's rows have landed (this wave's share) before the barrier. A wave's loads retire in order;
            // stores share the counter and are not ordered against loads, so the count allowed to remain is that of the
            // loads issued in this band body for a later band (AHEAD = 2), never more: an outstanding store then only
            // makes the wait longer.
            static_assert(AHEAD == 1 || AHEAD == 2, "the wait below counts this band's loads only");
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * NL) : "memory");
            barrier();
            if(b + 1 < nbands)
                static_for<MTW>([&](auto t_c) { read_one(std::integral_constant<int, PHN>{}, std::integral_constant<int, 0>{}, t_c); });
            if constexpr(!PIPE)
            {
                // (the MFMA results must have left the pipeline before the epilogue reads them: inline-assembly MFMAs are
                // invisible to the compiler's hazard handling)
                asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                if constexpr(DT == DT_I8 && decltype(epi_c)::value == EPI_REQUANT_RND)
                {
                    // The table epilogue two tiles at a time: the byte reads of tile t + 1 are on their way while tile t is
                    // packed and stored (LDS reads return in order: at most the next tile's 4 * NBT outstanding means this
                    // tile's have landed; the wait counter holds 15). With one wave per SIMD nothing else hides their latency.
                    const uint32_t lut_lds = ring_lds + (uint32_t)RING_BYTES;
                    const uint32_t soff    = (uint32_t)((n * p.Ho + TH * b) * p.Wo) * (KO * ES);
                    int bb[2][4 * NBT];
                    auto issue = [&](auto t_c) {
                        constexpr int t = decltype(t_c)::value;
#pragma unroll
                        for(int j = 0; j < NBT; ++j)
                        {
                            const acc_t v = acc0[t][j];
#pragma unroll
                            for(int i = 0; i < 4; ++i)
                                bb[t & 1][4 * j + i] = lds_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(p.scale_gemm * (float)v[i], 0u, lut_lds));
                        }
                    };
                    issue(std::integral_constant<int, 0>{});
                    static_for<MTW>([&](auto t_c) {
                        constexpr int t = decltype(t_c)::value;
                        if constexpr(t + 1 < MTW)
                        {
                            issue(std::integral_constant<int, t + 1>{});
                            asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(4 * NBT < 15 ? 4 * NBT : 15) : "memory");
                        }
                        else
                            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        __builtin_amdgcn_sched_barrier(0);
                        int o[NBT];
#pragma unroll
                        for(int j = 0; j < NBT; ++j)
                            o[j] = pack4_low_bytes(bb[t & 1][4 * j], bb[t & 1][4 * j + 1], bb[t & 1][4 * j + 2], bb[t & 1][4 * j + 3]);
                        static_assert(NBT == 4, "16 channels per lane");
                        store_out(i32x4{o[0], o[1], o[2], o[3]}, (int)rout[t] < p.Ho - TH * b ? ooff[t] : kOutOfRange, soff);
                        __builtin_amdgcn_sched_barrier(0);
                    });
                }
                else
                    static_for<MTW>([&](auto t_c) { store_tile(set_c, t_c, epi_c, n, b); });
            }
        };

        // the functor is dispatched once per image, outside the band loop
        // rows of the first band and of the AHEAD - 1 bands after it
        auto first_rows = [&](int n) {
            static_for<NEED + TH * (AHEAD - 1)>([&](auto j_c) {
                static_for<KSP>([&](auto h_c) { load_row(n, decltype(j_c)::value, j_c, h_c); });
            });
        };
        auto image = [&](auto epi_c, int n, bool first) {
            // (every wave has passed the barrier that ended the previous image.) Only the first band's rows have to land
            // before the MFMAs start: a wave's loads retire in order, and behind them are the later bands' rows and, in the
            // first image, the weights
            if(first)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * TH * KSP + TAPS * KSP * NBT) : "memory");
            else
            {
                first_rows(n);
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * TH * KSP) : "memory");
            }
            barrier();
            static_for<MTW>([&](auto t_c) { read_one(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, t_c); });
            // the band loop, unrolled over the ring's period (and, PIPE, the two accumulator sets): the band's position in
            // the ring is a compile-time constant of every read offset and load destination
            constexpr int NCOPY = PIPE && NPH % 2 ? 2 * NPH : NPH;
            int b = 0;
            for(;;)
            {
                bool done = false;
                static_for<NCOPY>([&](auto k_c) {
                    if(!done)
                    {
                        band(std::integral_constant<int, (decltype(k_c)::value % NPH) * TH>{},
                             std::integral_constant<int, PIPE ? decltype(k_c)::value % 2 : 0>{}, epi_c, n, b);
                        done = ++b == nbands;
                    }
                });
                if(done)
                    break;
            }
            if constexpr(PIPE)
            {
                // the last band's results
                asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                load_resi(n, nbands - 1);
                if((nbands - 1) & 1)
                    static_for<MTW>([&](auto t_c) { store_tile(std::integral_constant<int, 1>{}, t_c, epi_c, n, nbands - 1); });
                else
                    static_for<MTW>([&](auto t_c) { store_tile(std::integral_constant<int, 0>{}, t_c, epi_c, n, nbands - 1); });
            }
            barrier(); // the ring is free for the next image's first rows
        };
        using std::integral_constant;
        // the first image's rows are requested before the weights (the launcher starts no workgroup without an image)
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
            if constexpr(I8PERCH)
            {
                if(p.epi == EPI_RELU_MUL2_CLAMP)
                    image(integral_constant<int, EPI_RELU_MUL2_CLAMP>{}, n, first);
                else
                    image(integral_constant<int, EPI_MUL2_CLAMP>{}, n, first);
            }
            else if constexpr(DT == DT_I8)
            {
                if(p.epi == EPI_REQUANT_RND)
                    image(integral_constant<int, EPI_REQUANT_RND>{}, n, first);
                else if(p.epi == EPI_REQUANT_CK)
                    image(integral_constant<int, EPI_REQUANT_CK>{}, n, first);
                else
                    image(integral_constant<int, EPI_PASSTHROUGH>{}, n, first);
            }
            else if constexpr(FUSED)
            {
                if(p.epi == EPI_ADD_RELU_ADD)
                    image(integral_constant<int, EPI_ADD_RELU_ADD>{}, n, first);
                else
                    image(integral_constant<int, EPI_ADD_RELU>{}, n, first);
            }
            else
                image(integral_constant<int, EPI_PASSTHROUGH>{}, n, first);
        }
        // loads of rows past the last band still target this workgroup's LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
};

template <int DT, int MTW, bool FUSED>
__global__ __launch_bounds__(256) void conv_patch_kernel(const ConvPatchArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_patch_smem[];
    ConvPatch<DT, MTW, FUSED>::run(p, ckx_patch_smem);
}

// (conv_patch.hip) dt: DT_F16 / DT_I8; fused: the add / ReLU epilogues (fp16), per-channel requant scales (int8); Wo = 56
hipError_t launch_conv_patch(int dt, bool fused, const ConvPatchArgs& a, hipStream_t s);

} // namespace ckx
