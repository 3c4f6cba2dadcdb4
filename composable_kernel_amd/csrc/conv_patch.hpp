// Input-patch conv2d forward for gfx950, fp16 and int8, NHWC / KYXC / NHWK: the 3x3-class layers with few
// channels (ResNet conv2_x: C = 64, K = 64, 56 x 56), where the implicit-GEMM tile kernel re-reads
// every input pixel once per filter tap out of L2 and is bound by that.
//
// Takes the place of the same reference kernel as the tile kernel
// (DeviceConv2dFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K,
// device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:57-720) for the shapes it covers:
//   C = 64 (one pixel = one LDS row of 128 bytes fp16 / 64 bytes int8 = one tap's K tile), K = 64,
//   Y x X taps, stride 1, dilation 1, Wo = 8 * MTW <= 56, Wo + X - 1 <= 64.
// int8: one pixel is exactly one MFMA k-step (16x16x64), half the LDS reads and MFMAs per tap of fp16;
// the epilogue is the requant / PassThrough family of the GEMM, 8 consecutive int8 channels per lane.
//
//  * A workgroup (4 waves) owns whole images and walks them in bands of 4 output rows. The
//    input rows a band needs (4 + Y - 1) live in LDS in a RING of 10 rows x 64 pixels x 128 (64) B;
//    while band b is multiplied, the 4 new rows of band b + 1 are fetched into the ring slots
//    that band b - 1 has finished with. Every input pixel is read from memory ONCE.
//  * All Y * X * 64 weight rows (72 KB) are LDS-resident for the life of the workgroup.
//  * The A fragment of tap (y, x) for 16 consecutive output pixels is the patch shifted by
//    (y rows, x pixels): the same 128-byte rows, another base address. A lane keeps one
//    precomputed byte offset per (M tile, x) and one per (M tile, y): a fragment address is one add.
//  * 16-byte chunks are swizzled by the patch COLUMN (fp16: chunk ^ (col & 7); int8, 4 chunks per pixel:
//    chunk ^ (bit 0 and bit 2 of col)), so the 16 lanes the LDS serves in one cycle of a fragment read land on
//    different banks.
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
    MagicDiv div_wo;
    int epi; // fp16: EPI_PASSTHROUGH, EPI_ADD_RELU, EPI_ADD_RELU_ADD; int8: EPI_PASSTHROUGH, EPI_REQUANT_CK, EPI_REQUANT_RND,
             // EPI_MUL2_CLAMP / EPI_RELU_MUL2_CLAMP (one requant scale per output channel)
    const void* bias; // [64]: fp16 bias (fp16 kernels), fp32 requant scales (the int8 per-channel variant)
    const void* resi; // NHWK fp16
    float scale_gemm, scale_relu; // int8 requant epilogues
};

// FUSED: the add / ReLU epilogues (bias, residual) are compiled in; the plain instantiation keeps
// their registers free
// TH output rows per band, WMW x (4 / WMW) waves: a wave multiplies 16 * MTW pixels x 64 / (4 / WMW) channels.
// fp16: 4 rows, 2 x 2 waves (the LDS holds no deeper ring beside the weights); int8: 8 rows, 4 x 1 waves -- every
// wave then owns all 64 channels of its pixels (one 16-byte store per pixel and lane, whole 64-byte pixels per
// four lanes) and reads 11 fragments per 28 MFMAs instead of 9 per 14.
template <int DT, int MTW, int Y, int X, bool FUSED, int TH_ = (DT == DT_I8 ? 8 : 4), int WMW = (DT == DT_I8 ? 4 : 2)>
struct ConvPatch
{
    static constexpr int ES     = DT == DT_I8 ? 1 : 2;
    static constexpr int TH     = TH_;              // output rows per band
    static constexpr int WNW    = 4 / WMW;          // waves along the output channels
    static constexpr int NBT    = 4 / WNW;          // 16-channel weight tiles per wave (2 / 4)
    static constexpr int CPW    = 16 * NBT;         // channels per wave
    // bands of input rows in flight ahead of the band being multiplied. fp16 rows fill the LDS with one; int8
    // rows are half as large, and three bands of head start take the HBM latency out of the band loop (one
    // image per workgroup at a time: nothing else would hide it)
    static constexpr int AHEAD  = ES == 1 ? 2 : 1;
    static constexpr int RING   = (AHEAD + 1) * TH + 2; // ring rows (Y <= 3)
    static constexpr int PITCH  = 64;               // pixels per ring row
    static constexpr int PXB    = 64 * ES;          // bytes per pixel (C * element size)
    static constexpr int CPP    = PXB / 16;         // 16-byte chunks per pixel (8 / 4)
    static constexpr int PPI    = 64 / CPP;         // pixels (or weight rows) covered by one wave-wide direct load
    static constexpr int KSP    = PXB / 64;         // MFMA k-steps per tap (2 / 1)
    static constexpr int KO     = 64;               // output channels
    static constexpr int TAPS   = Y * X;
    static constexpr int RING_BYTES = RING * PITCH * PXB;
    static constexpr int WEI_BYTES  = TAPS * KO * PXB;
    static constexpr int LUT        = DT == DT_I8 ? 256 : 0; // table of the rounded requant epilogue, behind the weights
    static constexpr int LDS        = RING_BYTES + WEI_BYTES + LUT;
    static constexpr int NT         = 256;
    static constexpr int NEED_ROWS  = TH + Y - 1;   // input rows of one band
    static_assert(Y >= 1 && Y <= 3 && X >= 1 && X <= 3 && MTW >= 1 && MTW <= 7, "covered shapes");
    static_assert(DT == DT_F16 || DT == DT_I8, "fp16 (FUSED: the add / ReLU epilogues) or int8 (FUSED: per-channel requant)");
    static constexpr bool F16FUSED = FUSED && DT == DT_F16, I8PERCH = FUSED && DT == DT_I8;
    static_assert((WMW == 2 || WMW == 4) && (NBT == 2 || DT == DT_I8), "wave arrangements built");
    static_assert(LDS <= 160 * 1024, "ring + weights fit the LDS");
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    // swizzle key of a pixel column / weight row: the 16 rows of a fragment read must land on distinct banks
    // (a ds_read_b128 is served in four cycles; the 16 lanes of a cycle are those with equal (lane bit 5, parity of
    // lane bits 2..4). For 64-byte pixels the first choice, (r >> 2) & 3, left two-way conflicts under that grouping:
    // SQ_LDS_BANK_CONFLICT was half of SQ_LDS_IDX_ACTIVE)
    __device__ static __forceinline__ uint32_t key(uint32_t r) { return CPP == 8 ? (r & 7u) : ((r & 1u) | ((r >> 1) & 2u)); }

    __device__ static __forceinline__ void run(const ConvPatchArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const int wm = wave / WNW, wn = wave % WNW;
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        uint8_t* ring = smem;
        uint8_t* wlds = smem + RING_BYTES;

        const __amdgpu_buffer_rsrc_t rsrc_in  = make_rsrc(p.in, p.in_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_wei = make_rsrc(p.wei, p.wei_bytes);

        if constexpr(DT == DT_I8)
        {
            if(p.epi == EPI_REQUANT_RND)
                requant_lut_fill(smem + RING_BYTES + WEI_BYTES, p.scale_relu, (int)threadIdx.x, 256);
        }

        // ---- weights: LDS row tap*64 + r holds output channel w_row_to_ch(r), swizzled by r & 7
        {
            constexpr int BPT  = KO / PPI;                 // wave-wide loads per tap (8 / 4)
            const uint32_t rl  = (uint32_t)(lane / CPP);   // row within the block of PPI rows
            const uint32_t pos = (uint32_t)(lane % CPP);
            for(int k = wave; k < TAPS * BPT; k += 4)
            {
                const uint32_t tap = (uint32_t)k / BPT;
                const uint32_t r   = ((uint32_t)k % BPT) * PPI + rl; // 0..63
                // within a wave's group of CPW rows, row 16j + 4q + i holds channel 4*NBT*q + 4j + i
                const uint32_t rr = r % CPW;
                const uint32_t ch = (r - rr) + (4 * NBT) * ((rr >> 2) & 3u) + 4 * (rr >> 4) + (rr & 3u);
                const uint32_t voff = (ch * TAPS + tap) * PXB + ((pos ^ key(r)) << 4);
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
            ooff[t]          = ((r * (uint32_t)p.Wo + w) * KO + (uint32_t)(CPW * wn) + (uint32_t)(4 * NBT) * fq) * ES;
#pragma unroll
            for(int x = 0; x < X; ++x)
            {
                const uint32_t cc = w + (uint32_t)x;
                coff[t][x]        = cc * PXB + ((fq ^ key(cc)) << 4);
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
        // int8, per-channel requant: the scales of the lane's 4 * NBT consecutive channels, for the life of the workgroup
        float chsc[I8PERCH ? 4 * NBT : 1];
        if constexpr(I8PERCH)
        {
#pragma unroll
            for(int e = 0; e < 4 * NBT; ++e)
                chsc[e] = reinterpret_cast<const float*>(p.bias)[CPW * wn + 4 * NBT * (int)fq + e];
        }

        uint32_t boff[NBT]; // weight fragment of n-tile j, k-step 0, tap 0
#pragma unroll
        for(int j = 0; j < NBT; ++j)
            boff[j] = (uint32_t)(CPW * wn + 16 * j + (int)frow) * PXB + ((fq ^ key(frow)) << 4);

        // ---- input rows -> ring: block k = (row j, PPI-pixel column group cg) ------------------
        // lane: patch column PPI*cg + lane/CPP, LDS chunk position lane%CPP <- global chunk pos ^ key(col)
        constexpr int BPR = PITCH / PPI; // blocks per ring row (8 / 4)
        auto load_block = [&](int n, int j, int cg) {
            const int cc = PPI * cg + lane / CPP;
            const int wi = cc - p.pL, hi = j - p.pT;
            const bool ok = (uint32_t)hi < (uint32_t)p.Hi && (uint32_t)wi < (uint32_t)p.Wi && n < p.N;
            const uint32_t chunk = (uint32_t)(lane % CPP) ^ key((uint32_t)cc);
            const uint32_t voff =
                ((uint32_t)((n * p.Hi + hi) * p.Wi + wi) * PXB + (chunk << 4)) | (ok ? 0u : kOutOfRange);
            const int slot = j % RING;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_in, (lds_ptr_t)(ring + (size_t)(slot * PITCH + PPI * cg) * PXB),
                                                     16, voff, 0, 0, 0);
        };

        acc_t acc[MTW][NBT];
#pragma unroll
        for(int t = 0; t < MTW; ++t)
#pragma unroll
            for(int j = 0; j < NBT; ++j)
                acc[t][j] = acc_t{0, 0, 0, 0};

        auto barrier = [&]() {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        };

        uint32_t roff[MTW][Y];   // ring byte offset of (M tile's output row + y) for the current band
        uint32_t roff_n[MTW][Y]; // ... for the next band: worked out one value per MFMA group, in the MFMAs' shadow
        i32x4 af[2][MTW], bf[2][NBT];
        const int nbands = (p.Ho + TH - 1) / TH;
        for(int n = (int)blockIdx.x; n < p.N; n += (int)gridDim.x)
        {
            // rows of the first band (every wave has passed the barrier that ended the previous image)
            // and of the AHEAD - 1 bands after it; only the first band's have to land before the MFMAs start (a wave
            // issues its blocks in ascending order and loads retire in order)
            static_assert((NEED_ROWS * BPR) % 4 == 0 && (TH * BPR) % 4 == 0, "the same number of blocks for every wave");
            for(int k = wave; k < (NEED_ROWS + TH * (AHEAD - 1)) * BPR; k += 4)
                load_block(n, k / BPR, k % BPR);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * TH * BPR / 4) : "memory");
            barrier();

            for(int b = 0; b < nbands; ++b)
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

                // fragment r of k-step s = (tap, half) (int8: s = tap): r = 0, 1 the two weight tiles, then the
                // M tiles in the order in which the MFMAs use them
                auto read_one = [&](int s, int r) {
                    const int buf = s & 1, tap = s / KSP, ks = s % KSP, y = tap / X, x = tap % X;
                    if(r < NBT)
                        bf[buf][r] = *reinterpret_cast<const i32x4*>(wlds + tap * (KO * PXB) +
                                                                     (boff[r] ^ (uint32_t)(ks * 64)));
                    else
                        af[buf][r - NBT] = *reinterpret_cast<const i32x4*>(ring + roff[r - NBT][y] +
                                                                           (coff[r - NBT][x] ^ (uint32_t)(ks * 64)));
                };
                auto mfma_pair = [&](int s, int t) {
                    const int buf = s & 1;
#pragma unroll
                    for(int j = 0; j < NBT; ++j)
                    {
                        if constexpr(DT == DT_I8)
                            acc[t][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[buf][j], af[buf][t], acc[t][j], 0, 0, 0);
                        else
                            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bf[buf][j]),
                                                                            __builtin_bit_cast(f16x8, af[buf][t]),
                                                                            acc[t][j], 0, 0, 0);
                    }
                };

                if(b == 0)
                {
#pragma unroll
                    for(int r = 0; r < MTW + NBT; ++r)
                        read_one(0, r);
                }
                // residual values of this band: plain loads, issued before the band's direct loads and
                // waited for with them (a load issued after the stores would have to wait for those)
                if constexpr(F16FUSED)
                  if(has_resi)
                {
                    const uint8_t* resi_band = reinterpret_cast<const uint8_t*>(p.resi) +
                                               ((size_t)n * p.Ho + (size_t)TH * b) * p.Wo * (KO * sizeof(_Float16));
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
                        if(TH * b + (int)rout[t] < p.Ho)
                            resi8[F16FUSED ? t : 0] = *reinterpret_cast<const f16x8*>(resi_band + ooff[t]);
                }
                // One k-step = MTW groups pinned in source order: [reads of the NEXT k-step, spread over
                // the first groups and finished two groups early] [one direct load of the next band's
                // rows] [the 2 MFMAs of one M tile]. With one wave per SIMD nothing else hides the
                // issue slots of the reads, so they go between the MFMAs.
                const uint32_t j1mod = (uint32_t)((j0 + TH) % RING); // first ring row of the next band
                static_assert(KSP * TAPS >= Y, "one k-step per filter row for the next band's ring offsets");
                constexpr int NR = MTW + NBT, RG = MTW > 2 ? MTW - 2 : MTW;
                constexpr int NS = KSP * TAPS;           // k-steps of a band
                constexpr int NBLK = TH * BPR / 4;       // direct loads per wave for the next band's rows
                static_assert(NBLK <= NS, "one direct load per k-step");
#pragma unroll
                for(int s = 0; s < NS; ++s)
                {
#pragma unroll
                    for(int g = 0; g < MTW; ++g)
                    {
                        if(s + 1 < NS)
                        {
#pragma unroll
                            for(int r = (g < RG ? g : RG) * NR / RG; r < (g + 1 < RG ? g + 1 : RG) * NR / RG; ++r)
                                read_one(s + 1, r);
                        }
                        // the 4 new input rows of the next band: TH * BPR blocks, NBLK per wave, one per k-step
                        if(s < NBLK && g == MTW - 1)
                        {
                            const int k = wave + 4 * s;
                            load_block(n, j0 + NEED_ROWS + TH * (AHEAD - 1) + k / BPR, k % BPR);
                        }
                        // ring offsets of the next band's rows, one (M tile, y) per group of the first Y k-steps
                        if(s < Y)
                        {
                            uint32_t sl  = j1mod + rout[g] + (uint32_t)s;
                            sl           = sl >= (uint32_t)RING ? sl - RING : sl;
                            roff_n[g][s] = sl * (PITCH * PXB);
                        }
                        mfma_pair(s, g);
                        // Order inside the group: MFMA, one address add, one fragment read, MFMA, ... With one wave per
                        // SIMD only about 12 of an MFMA's 16 cycles hide other issue: a run of adds and reads ahead of
                        // the MFMAs leaves the matrix pipe idle (a loop of [add add read read, 4 MFMAs] issues MFMAs at
                        // 78 % of the back-to-back rate, [MFMA add read MFMA add read MFMA MFMA] at 92 %).
                        // (int8 only: 40.8 against 41.5 us on the 56 x 56 layer; the fp16 kernel, two MFMAs per group, measured
                        // 2 % slower with it)
                        if constexpr(DT == DT_I8)
#pragma unroll
                        for(int j = 0; j < NBT; ++j)
                        {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
                            __builtin_amdgcn_sched_group_barrier(0x002, 1, 0); // VALU
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // LDS read
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }

                // the next band's rows have landed (this wave's share) before the stores go out. Loads retire in
                // order among themselves, so "at most the loads of the AHEAD - 1 later bands outstanding" implies
                // it; stores share the counter and are not ordered against loads, which can only make this
                // wait longer, never too short
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * NBLK) : "memory");
                // every wave is through with this band's rows, and the next band's rows are visible:
                // its first fragments are read under the epilogue
                barrier();
                if(b + 1 < nbands)
                {
#pragma unroll
                    for(int t = 0; t < MTW; ++t)
#pragma unroll
                        for(int y = 0; y < Y; ++y)
                            roff[t][y] = roff_n[t][y];
#pragma unroll
                    for(int r = 0; r < MTW + NBT; ++r)
                        read_one(0, r);
                }

                // ---- epilogue: 8 consecutive channels of one pixel per lane and M tile ----------
                uint8_t* out_band = reinterpret_cast<uint8_t*>(p.out) + ((size_t)n * p.Ho + (size_t)TH * b) * p.Wo * (KO * ES);
                if constexpr(DT == DT_I8)
                {
                    // 8 consecutive int8 channels per lane and M tile: the requant / PassThrough family of the GEMM
                    // epilogue. The mode is dispatched ONCE per band (a compile-time parameter of the body): tested
                    // per value it turns the epilogue into hundreds of scalar branches, which cost more than the
                    // whole K loop.
                    auto store_band = [&](auto epi_c) {
                        constexpr int EPI = decltype(epi_c)::value;
#pragma unroll
                        for(int t = 0; t < MTW; ++t)
                        {
                            if(TH * b + (int)rout[t] < p.Ho)
                            {
                                int o[NBT];
                                if constexpr(EPI == EPI_MUL2_CLAMP || EPI == EPI_RELU_MUL2_CLAMP)
                                {
                                    constexpr bool relu = EPI == EPI_RELU_MUL2_CLAMP;
                                    constexpr int NS    = I8PERCH ? 4 * NBT : 1;
#pragma unroll
                                    for(int j = 0; j < NBT; ++j)
                                        o[j] = pack4_low_bytes(mul2_clamp(acc[t][j][0], chsc[(4 * j) % NS], relu),
                                                               mul2_clamp(acc[t][j][1], chsc[(4 * j + 1) % NS], relu),
                                                               mul2_clamp(acc[t][j][2], chsc[(4 * j + 2) % NS], relu),
                                                               mul2_clamp(acc[t][j][3], chsc[(4 * j + 3) % NS], relu));
                                }
                                else if constexpr(EPI == EPI_REQUANT_RND)
                                {
                                    i32x4 v[NBT];
#pragma unroll
                                    for(int j = 0; j < NBT; ++j)
                                        v[j] = acc[t][j];
                                    int bb[4 * NBT];
                                    requant_lut<NBT>(v, p.scale_gemm,
                                                     (uint32_t)(uintptr_t)(lds_ptr_t)smem + (uint32_t)(RING_BYTES + WEI_BYTES), bb);
#pragma unroll
                                    for(int j = 0; j < NBT; ++j)
                                        o[j] = pack4_low_bytes(bb[4 * j], bb[4 * j + 1], bb[4 * j + 2], bb[4 * j + 3]);
                                }
                                else
                                {
#pragma unroll
                                    for(int j = 0; j < NBT; ++j)
                                        o[j] = pack4_low_bytes(epilogue_i8<EPI>(acc[t][j][0], p.scale_gemm, p.scale_relu),
                                                               epilogue_i8<EPI>(acc[t][j][1], p.scale_gemm, p.scale_relu),
                                                               epilogue_i8<EPI>(acc[t][j][2], p.scale_gemm, p.scale_relu),
                                                               epilogue_i8<EPI>(acc[t][j][3], p.scale_gemm, p.scale_relu));
                                }
                                if constexpr(NBT == 4)
                                    *reinterpret_cast<i32x4*>(out_band + ooff[t]) = i32x4{o[0], o[1], o[2], o[3]};
                                else
                                    *reinterpret_cast<i32x2*>(out_band + ooff[t]) = i32x2{o[0], o[1]};
                            }
#pragma unroll
                            for(int j = 0; j < NBT; ++j)
                                acc[t][j] = acc_t{0, 0, 0, 0};
                        }
                    };
                    if constexpr(I8PERCH)
                    {
                        if(p.epi == EPI_RELU_MUL2_CLAMP)
                            store_band(std::integral_constant<int, EPI_RELU_MUL2_CLAMP>{});
                        else
                            store_band(std::integral_constant<int, EPI_MUL2_CLAMP>{});
                    }
                    else if(p.epi == EPI_REQUANT_RND)
                        store_band(std::integral_constant<int, EPI_REQUANT_RND>{});
                    else if(p.epi == EPI_REQUANT_CK)
                        store_band(std::integral_constant<int, EPI_REQUANT_CK>{});
                    else
                        store_band(std::integral_constant<int, EPI_PASSTHROUGH>{});
                }
                else
                {
                    // (fused variant: the functor is a compile-time parameter of the body as well)
                    auto store_band = [&](auto epi_c) {
                        constexpr int EPI = decltype(epi_c)::value;
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
                                    if constexpr(EPI != EPI_PASSTHROUGH)
                                    {
                                        v0 = epi_f16_value(EPI, v0, (float)bias8[i], (float)resi8[FUSED ? t : 0][i]);
                                        v1 = epi_f16_value(EPI, v1, (float)bias8[4 + i], (float)resi8[FUSED ? t : 0][4 + i]);
                                    }
                                    o[i]     = (_Float16)v0;
                                    o[4 + i] = (_Float16)v1;
                                }
                                *reinterpret_cast<f16x8*>(out_band + ooff[t]) = o;
                            }
                            acc[t][0] = acc[t][1] = acc_t{0, 0, 0, 0};
                        }
                    };
                    if constexpr(FUSED)
                    {
                        if(p.epi == EPI_ADD_RELU_ADD)
                            store_band(std::integral_constant<int, EPI_ADD_RELU_ADD>{});
                        else
                            store_band(std::integral_constant<int, EPI_ADD_RELU>{});
                    }
                    else
                        store_band(std::integral_constant<int, EPI_PASSTHROUGH>{});
                }
            }
            barrier(); // the ring is free for the next image's first rows
        }
        // the weight loads of a workgroup that got no image still target its LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
};

template <int DT, int MTW, int Y, int X, bool FUSED>
__global__ __launch_bounds__(256) void conv_patch_kernel(const ConvPatchArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_patch_smem[];
    ConvPatch<DT, MTW, Y, X, FUSED>::run(p, ckx_patch_smem);
}

} // namespace ckx
