// 256 x 256 C tile computed by FOUR waves -- one per SIMD, wave tile 128 x 128 -- for dense K-contiguous GEMMs
// (A row-major, B column-major, optionally a strided batch of them), one K run.
//
// Same data path as gemm_tile.hpp (128-byte K tiles, direct global->LDS loads with the XOR swizzle and the B row
// permutation applied by the choice of each lane's global chunk, D^T = B_frag x A_frag, register epilogue), a different
// division of labour:
//  * one wave per SIMD. Two waves of one SIMD do not interleave evenly: the older one runs ahead, issues its direct
//    loads early, the younger one issues its loads late and everybody waits for those at the next barrier. With a
//    single wave per SIMD the loads of all four waves go out at the same point of the iteration. (An instruction-mix
//    model of both loops with real operand traffic: 19.7 cycles per MFMA with two waves per SIMD, 17.8 with one.)
//  * nothing but MFMAs, fragment reads and loads in the K loop: a VALU instruction between the MFMAs of a SIMD's only
//    wave costs about seven cycles of the matrix pipeline (nothing else runs meanwhile), so the loads' offsets are fixed
//    registers and the K tile's offset travels in the scalar offset.
//  * 128 x 128 wave tiles: 16 fragment reads per 64 MFMAs instead of 12 per 32.
//  * the accumulators live in AccVGPRs (224 of a lane's 256; the last fragment row's in VGPRs): the MFMAs are inline
//    assembly with the accumulator tied ("+a"), which is what keeps the register allocator from shuffling them through
//    VGPRs; the 128 VGPRs of the two fragment sets (register double buffer over the two k-steps of a K tile), the 16
//    load offsets and the addresses fit the architectural half.
//  * 16-bit outputs leave in 64-byte runs per row and store instruction (row_to_col).
// The K loop is a loop of its own inside the loop over tiles, without prefetch across tiles: a workgroup normally has
// one tile; the eight-wave tile kernel keeps the problems whose epilogues or operand layouts this one does not have.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

// FUSED (fp16): the epilogues with D operands (add / ReLU functors, Bilinear, AddAddFastGelu) as a kernel of their own,
// like the FUSED variants of the tile kernel.
// EPI (int8, plain epilogues): the requant form as a compile-time constant, so that the last K tile's loop, which stores
// finished fragment rows between its MFMAs, carries no branch on it.
template <int DT, bool FUSED = false, int EPI = EPI_PASSTHROUGH>
struct GemmW4
{
    static_assert(!FUSED || DT == DT_F16, "D-operand epilogues: fp16");
    static_assert(EPI == EPI_PASSTHROUGH || (DT == DT_I8 && (EPI == EPI_REQUANT_CK || EPI == EPI_REQUANT_RND)), "");
    static constexpr int BM = 256, BN = 256, BKB = 128, NW = 4, NT = NW * 64, NST = 2;
    static constexpr int ES     = DT == DT_I8 ? 1 : 2;
    static constexpr int A_TILE = BM * BKB, B_TILE = BN * BKB, STAGE = A_TILE + B_TILE;
    static constexpr int LUT    = DT == DT_I8 ? 256 : 0;
    static constexpr int LDS    = NST * STAGE + LUT;
    static constexpr int MT = 8, NB = 8;  // A fragments (16 rows each) and B fragments (16 columns each) of a wave per k-step
    static constexpr int NLA = 8, NLB = 8, LPT = NLA + NLB; // 16-byte direct loads per thread and K tile
    static constexpr int NMH = MT * NB;   // MFMAs per half-iteration (one k-step)
    // LDS: [A stage 0 | A stage 1 | B stage 0 | B stage 1 | requant table]. Both stages of an operand lie within the
    // 16-bit offset field of a fragment read, so a lane's four read addresses (A / B x k-step) serve both stages.
    static constexpr int A_AT(int st) { return st * A_TILE; }
    static constexpr int B_AT(int st) { return NST * A_TILE + st * B_TILE; }
    // A direct load's immediate offset moves its LDS address AND its global address. A wave's eight load slots of an
    // operand are 1 KB apart in LDS, so one M0 value serves four loads (immediates 0 .. 3 KB); the per-lane global
    // offsets carry kImmBias minus the immediate, and the buffer resources start kImmBias bytes before the operands.
    static constexpr int kImmBias = 3072;
    // M0 for load slot SLOT (and the three after it) of stage ST, relative to the wave's first slot in A stage 0; a
    // stage that is only known at run time (ST < 0) is added to the base register instead (A_TILE == B_TILE)
    static constexpr int m0_add(int slot, int st)
    {
        return (slot < NLA ? A_AT(st < 0 ? 0 : st) : B_AT(st < 0 ? 0 : st)) + ((slot % NLA) / 4) * 4096;
    }
    template <typename ST>
    static constexpr int stage_ct(ST)
    {
        if constexpr(std::is_same<ST, int>::value)
            return -1;
        else
            return ST::value;
    }
    template <typename ST>
    __device__ static __forceinline__ uint32_t stage_rt(ST st)
    {
        if constexpr(std::is_same<ST, int>::value)
            return (uint32_t)st * A_TILE;
        else
            return 0u;
    }
    // SPREAD: the B half of the K tile after next is requested during the FIRST half of an iteration (behind a
    // second barrier, once every wave has the current tile's B fragments of k-step 1), the A half during the second:
    // the CU's address unit sees eight loads per wave and half instead of sixteen in one.
#ifndef CKX_W4_SPREAD
#define CKX_W4_SPREAD 2
#endif
    static constexpr bool SPREAD = CKX_W4_SPREAD != 0;
    // first half of a SPREAD iteration: a B read behind every H0_RB-th MFMA, wait + barrier behind MFMA H0_BAR, B loads
    // behind MFMAs H0_L0 + i * H0_LS, A reads behind MFMAs H0_RA0 + i * H0_RAS
    static constexpr int H0_RB  = CKX_W4_SPREAD == 2 ? 1 : 2;
    static constexpr int H0_BAR = CKX_W4_SPREAD == 2 ? 13 : 23;
    static constexpr int H0_L0 = H0_BAR + 1, H0_LS = CKX_W4_SPREAD == 2 ? 6 : 5;
    static constexpr int H0_RA0 = H0_BAR + 3, H0_RAS = CKX_W4_SPREAD == 2 ? 5 : 4;
    static_assert(H0_L0 + (NLB - 1) * H0_LS < MT * NB && H0_RA0 + (MT - 1) * H0_RAS < MT * NB - 4 && NB * H0_RB <= H0_BAR, "");
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;

    // (the accumulators of the last fragment row stay in VGPRs: with all 256 AccVGPRs tied the allocator has no
    // register left to move one through and spills)
    // FIRST: the accumulator starts at zero (the literal 0 as the addend) instead of being read -- the first k-step of
    // a tile, which saves zeroing 256 registers per lane beforehand
    // M0ADD >= 0: the statement first writes M0 = m0_base + M0ADD for the direct loads that follow it (the MFMA is the
    // instruction the hazard wants between an M0 write and the load that uses it; as statements of their own the
    // compiler puts an s_nop in front of every such write).
    template <bool IN_VGPR, bool FIRST, int M0ADD = -1>
    __device__ static __forceinline__ void mfma(acc_t& c, const i32x4& b, const i32x4& a, uint32_t m0_base = 0)
    {
#define CKX_W4_MFMA(OP)                                                                                           \
    if constexpr(M0ADD >= 0)                                                                                      \
    {                                                                                                             \
        if constexpr(IN_VGPR && FIRST)                                                                            \
            asm volatile("s_add_u32 m0, %3, %4\n\t" OP " %0, %1, %2, 0" : "=v"(c) : "v"(b), "v"(a), "s"(m0_base), "n"(M0ADD) : "scc"); \
        else if constexpr(IN_VGPR)                                                                                \
            asm volatile("s_add_u32 m0, %3, %4\n\t" OP " %0, %1, %2, %0" : "+v"(c) : "v"(b), "v"(a), "s"(m0_base), "n"(M0ADD) : "scc"); \
        else if constexpr(FIRST)                                                                                  \
            asm volatile("s_add_u32 m0, %3, %4\n\t" OP " %0, %1, %2, 0" : "=a"(c) : "v"(b), "v"(a), "s"(m0_base), "n"(M0ADD) : "scc"); \
        else                                                                                                      \
            asm volatile("s_add_u32 m0, %3, %4\n\t" OP " %0, %1, %2, %0" : "+a"(c) : "v"(b), "v"(a), "s"(m0_base), "n"(M0ADD) : "scc"); \
    }                                                                                                             \
    else if constexpr(IN_VGPR && FIRST)                                                                           \
        asm volatile(OP " %0, %1, %2, 0" : "=v"(c) : "v"(b), "v"(a));                                             \
    else if constexpr(IN_VGPR)                                                                                    \
        asm volatile(OP " %0, %1, %2, %0" : "+v"(c) : "v"(b), "v"(a));                                            \
    else if constexpr(FIRST)                                                                                      \
        asm volatile(OP " %0, %1, %2, 0" : "=a"(c) : "v"(b), "v"(a));                                             \
    else                                                                                                          \
        asm volatile(OP " %0, %1, %2, %0" : "+a"(c) : "v"(b), "v"(a));
        if constexpr(DT == DT_I8)
        {
            CKX_W4_MFMA("v_mfma_i32_16x16x64_i8")
        }
        else if constexpr(DT == DT_BF16)
        {
            CKX_W4_MFMA("v_mfma_f32_16x16x32_bf16")
        }
        else
        {
            CKX_W4_MFMA("v_mfma_f32_16x16x32_f16")
        }
#undef CKX_W4_MFMA
    }

    // The four accumulator tuples of column group g of one fragment row, as VGPR values. Read out of the AccVGPRs by
    // inline assembly, in program order, one group at a time: left to itself the compiler reads all 224 of them at the
    // top of the epilogue and the allocator, short of 200 VGPRs there, spills fragment registers inside the K loop.
    template <bool IN_VGPR>
    __device__ static __forceinline__ void fetch_acc(std::integral_constant<bool, IN_VGPR>, const acc_t (&row)[NB], int g,
                                                     acc_t (&v)[4])
    {
#pragma unroll
        for(int t = 0; t < 4; ++t)
        {
            if constexpr(IN_VGPR)
                v[t] = row[g * 4 + t];
            else
            {
#pragma unroll
                for(int j = 0; j < 4; ++j)
                {
                    decltype(row[0][0] + 0) x;
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(row[g * 4 + t][j]));
                    v[t][j] = x;
                }
            }
        }
    }

    // LDS row of the staged B tile -> column of the tile. int8: b_row_to_col, a lane ends with 16 consecutive columns
    // (one 16-byte store, four lanes = 64 contiguous bytes of a row). 16-bit outputs: within a 64-column group, MFMA tile
    // t, MFMA row j = 4q + jj holds column 32 * (t / 2) + 8 * q + 4 * (t % 2) + jj, so the lane in 16-lane row q ends with
    // columns 8q .. 8q + 7 (tiles 0, 1) and 32 + 8q .. 32 + 8q + 7 (tiles 2, 3): each of its two 16-byte stores joins
    // those of the three other lanes of the row into 64 contiguous bytes, where 16 consecutive columns per lane would
    // interleave the two stores' 16-byte pieces.
    __device__ static __forceinline__ uint32_t row_to_col(uint32_t r)
    {
        if constexpr(DT == DT_I8)
            return b_row_to_col(r);
        else
        {
            const uint32_t t = (r >> 4) & 3u, q = (r & 15u) >> 2, jj = r & 3u;
            return (r & ~63u) | ((t >> 1) << 5) | (q << 3) | ((t & 1u) << 2) | jj;
        }
    }
    // the lane's 16 outputs of one row and 64-column group (first column n64) as two runs of 8 consecutive 16-bit values
    template <typename T>
    __device__ static __forceinline__ void store_2x8(T* crow, int n64, int q, int N, bool vec_ok, const f32x4 (&v)[4], bool nt)
    {
        typedef T tx8 __attribute__((ext_vector_type(8)));
#pragma unroll
        for(int h = 0; h < 2; ++h)
        {
            const int n0 = n64 + 32 * h + 8 * q;
            if(vec_ok && n0 + 8 <= N)
            {
                tx8 x;
#pragma unroll
                for(int j = 0; j < 4; ++j)
                    x[j] = (T)v[2 * h][j], x[4 + j] = (T)v[2 * h + 1][j];
                store_vec(reinterpret_cast<tx8*>(crow + n0), x, nt);
            }
            else
            {
#pragma unroll
                for(int e = 0; e < 8; ++e)
                    if(n0 + e < N)
                        crow[n0 + e] = (T)v[2 * h + e / 4][e % 4];
            }
        }
    }

    // 16 consecutive int8 outputs of one row from their (already requantised) values b[0..15]
    __device__ static __forceinline__ void store_bytes16(int8_t* crow, int n0, int N, bool vec_ok, const int* b, bool nt)
    {
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

    __device__ static __forceinline__ void run(const GemmArgs& p, uint8_t* smem)
    {
        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave >> 1, wn = wave & 1;
        const int nbatch      = p.batch > 0 ? p.batch : 1;
        const int ntiles      = p.tiles_m * p.tiles_n * nbatch; // C tiles of all batches, dealt to the XCDs batch by batch
        const uint32_t kbytes = (uint32_t)p.K * ES;
        const int nk_real     = (int)((kbytes + BKB - 1) / BKB);
        // (the plain epilogues run inside an iteration of their own, the last one: at least two K tiles, the second one
        // all zeros if need be)
        const int nk = nk_real > (FUSED ? 0 : 1) ? nk_real : (FUSED ? 1 : 2);

        const __amdgpu_buffer_rsrc_t rsrc_a =
            make_rsrc(reinterpret_cast<const uint8_t*>(p.a) - kImmBias, p.a_bytes + (uint32_t)kImmBias);
        const __amdgpu_buffer_rsrc_t rsrc_b =
            make_rsrc(reinterpret_cast<const uint8_t*>(p.b) - kImmBias, p.b_bytes + (uint32_t)kImmBias);
        const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
        if constexpr(DT == DT_I8 && EPI == EPI_REQUANT_RND) // (visible to every wave after the first barrier of the K loop)
            requant_lut_fill(smem + NST * STAGE, p.scale_relu, tid, NT);

        // slot j of a wave fills LDS rows (wave * 8 + j) * 8 + lane / 8 of the A (B) tile, chunk position lane % 8 with
        // chunk (lane % 8) ^ (row & 7) of that row
        const uint32_t kb = ((uint32_t)(lane & 7) ^ (uint32_t)((lane >> 3) & 7)) << 4;
        // LDS address of the wave's first load slot in A stage 0 (a scalar: M0 is this plus a constant)
        const uint32_t m0_base = smem_lds + (uint32_t)wave * (NLA * 1024);
        // fragment addresses: row = wave rows + 16 * fragment + lane % 16, chunk 4 * ks + lane / 16
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);
        auto frag_part      = [&](int row0, int ks) {
            return (uint32_t)(row0 + (int)frow) * BKB + ((((uint32_t)ks * 4 + fq) ^ (frow & 7u)) << 4);
        };
        const uint32_t fa[2] = {smem_lds + frag_part(wm * 128, 0), smem_lds + frag_part(wm * 128, 1)};
        const uint32_t fb[2] = {smem_lds + B_AT(0) + frag_part(wn * 128, 0), smem_lds + B_AT(0) + frag_part(wn * 128, 1)};

        const bool vec_ok = ((reinterpret_cast<uintptr_t>(p.c) | ((uintptr_t)p.ldc * ES) |
                              (nbatch > 1 ? (uintptr_t)p.bsc * ES : 0)) & 15u) == 0;
        const bool nt     = p.nt_store != 0;

        for(int unit = (int)blockIdx.x; unit < ntiles; unit += (int)gridDim.x)
        {
            int tm, tn, bi;
            tile_of_block(unit, p.tiles_m, p.tiles_n, nbatch, bi, tm, tn);
            const uint32_t a_batch = (uint32_t)((long)bi * p.bsa * ES), b_batch = (uint32_t)((long)bi * p.bsb * ES);
            uint8_t* const c_batch = reinterpret_cast<uint8_t*>(p.c) + (size_t)bi * p.bsc * ES;
            uint32_t a_off[NLA], b_off[NLB];
#pragma unroll
            for(int j = 0; j < NLA; ++j)
            {
                const uint32_t r    = (uint32_t)((wave * NLA + j) * 8 + (lane >> 3));
                const uint32_t gm   = (uint32_t)tm * BM + r;
                const uint32_t gn   = (uint32_t)tn * BN + row_to_col(r);
                const uint32_t bias = kb + (uint32_t)(kImmBias - (j & 3) * 1024);
                a_off[j]            = gm < (uint32_t)p.M ? a_batch + gm * (uint32_t)p.lda * ES + bias : kOutOfRange;
                b_off[j]            = gn < (uint32_t)p.N ? b_batch + gn * (uint32_t)p.ldb * ES + bias : kOutOfRange;
            }
            // One direct load, as inline assembly (the compiler's form writes M0 and a hazard nop before every load):
            // slot < NLA an A row group, else a B row group, of the K tile at byte offset k0, into the stage M0 points
            // into: M0 = m0_of(stage) + m0_add(slot) serves four consecutive slots, and is written by the statement of
            // the MFMA in front of the first of them (or, in the prologue, by a statement of its own). k0 travels in the
            // scalar offset, which the address uses and the range check does not: the per-lane offset alone decides
            // between the row (in range) and zeros (row past M / N: top bit). MASKED adds the top bit for chunks past K
            // and K tiles past the end -- a VALU instruction per load that the K tiles in the middle of the loop do
            // without (a VALU instruction between the MFMAs of a SIMD's only wave costs about seven cycles of the matrix
            // pipeline).
            auto load_slot = [&](auto slot_c, auto masked, uint32_t k0, uint32_t k_oob) {
                constexpr int SLOT = decltype(slot_c)::value, J = SLOT % NLA;
                const uint32_t off  = SLOT < NLA ? a_off[J] : b_off[J];
                const uint32_t voff = decltype(masked)::value ? (off | k_oob) : off;
                const __amdgpu_buffer_rsrc_t rsrc = SLOT < NLA ? rsrc_a : rsrc_b;
                asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds" ::"v"(voff), "s"(rsrc), "s"(k0),
                             "n"((J % 4) * 1024));
            };
            auto k_oob_of = [&](int kt) { return ((uint32_t)kt * BKB + kb < kbytes && kt < nk) ? 0u : kOutOfRange; };

            acc_t acc[MT][NB]; // (defined by the first k-step's MFMAs)

            // The previous tile's fragment reads are complete (its loop ends with a wait) but other waves may still be
            // reading: one barrier before the stages are refilled. Its C stores share the load counter and are not
            // ordered against loads: drained here, so that the counted wait below sees loads only.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            static_for<NST>([&](auto st_c) {
                const uint32_t oob = k_oob_of(decltype(st_c)::value);
                static_for<LPT>([&](auto s_c) {
                    if constexpr(decltype(s_c)::value % 4 == 0) // (one instruction between an M0 write and its load)
                        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0" ::"s"(m0_base),
                                     "n"(m0_add(decltype(s_c)::value, decltype(st_c)::value))
                                     : "scc");
                    load_slot(s_c, std::true_type{}, (uint32_t)decltype(st_c)::value * BKB, oob);
                });
            });
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPT) : "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");

            i32x4 af0[MT], bf0[NB], af1[MT], bf1[NB];
            // fragment r of k-step KS of stage ST: the B fragments first, then the A fragments
            auto read_one = [&](auto st, auto ks_c, auto r_c, i32x4(&af)[MT], i32x4(&bf)[NB]) {
                constexpr int KS = decltype(ks_c)::value, R = decltype(r_c)::value;
                if constexpr(std::is_same<decltype(st), int>::value)
                {
                    if constexpr(R < NB)
                        bf[R] = lds_read_b128<R * 16 * BKB>(fb[KS] + (uint32_t)st * B_TILE);
                    else
                        af[R - NB] = lds_read_b128<(R - NB) * 16 * BKB>(fa[KS] + (uint32_t)st * A_TILE);
                }
                else
                {
                    constexpr int ST = decltype(st)::value;
                    if constexpr(R < NB)
                        bf[R] = lds_read_b128<B_AT(ST) - B_AT(0) + R * 16 * BKB>(fb[KS]);
                    else
                        af[R - NB] = lds_read_b128<A_AT(ST) + (R - NB) * 16 * BKB>(fa[KS]);
                }
            };
            static_for<MT + NB>([&](auto r_c) {
                read_one(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, r_c, af0, bf0);
            });

            // One half of an iteration: the 64 MFMAs of one k-step on the fragments (caf, cbf); the 16 fragment reads of
            // the next k-step (k-step NKS of stage NST_) into (naf, nbf); direct loads of the K tile after next into
            // stage LST, whose fragments (of the operand being loaded) are all in registers by then.
            //   plain: no loads in the first half; all 16 in the second, one behind every fourth MFMA; reads behind
            //          every third MFMA (done after three quarters of the half);
            //   SPREAD, first half: the B reads behind every second MFMA, wait + barrier behind MFMA 23, then the eight B
            //          loads (one per five MFMAs) and the A reads; second half: the eight A loads, one per eight MFMAs.
            auto half_step = [&](auto first, auto second_half, auto masked, uint32_t k0, uint32_t k_oob, auto lst_c,
                                 const i32x4(&caf)[MT], const i32x4(&cbf)[NB], auto nst_c, auto nks, i32x4(&naf)[MT],
                                 i32x4(&nbf)[NB]) {
                constexpr bool H1 = decltype(second_half)::value;
                static_for<NMH>([&](auto m_c) {
                    constexpr int m = decltype(m_c)::value;
                    // (B fragments in snake order: across a change of the A fragment the other operand stays put)
                    constexpr int fi = m / NB, ft = (fi & 1) ? NB - 1 - m % NB : m % NB;
                    // which load slot, if any, goes out behind this MFMA
                    constexpr int slot = !SPREAD ? ((H1 && m % 4 == 0) ? m / 4 : -1)
                                         : H1    ? (m % 8 == 0 ? m / 8 : -1)
                                                 : ((m >= H0_L0 && (m - H0_L0) % H0_LS == 0 && (m - H0_L0) / H0_LS < NLB)
                                                        ? NLA + (m - H0_L0) / H0_LS
                                                        : -1);
                    constexpr int LST = stage_ct(decltype(lst_c){});
                    if constexpr(slot >= 0 && slot % 4 == 0)
                        mfma<fi == MT - 1, decltype(first)::value, m0_add(slot < 0 ? 0 : slot, LST)>(acc[fi][ft], cbf[ft], caf[fi],
                                                                                                m0_base + stage_rt(lst_c));
                    else
                        mfma<fi == MT - 1, decltype(first)::value>(acc[fi][ft], cbf[ft], caf[fi]);
                    if constexpr(slot >= 0)
                        load_slot(std::integral_constant<int, (slot < 0 ? 0 : slot)>{}, masked, k0, k_oob);
                    // which fragment read, if any, follows it
                    constexpr int rd = (!SPREAD || H1) ? ((m % 3 == 2 && m / 3 < MT + NB) ? m / 3 : -1)
                                       : m < NB * H0_RB ? ((m % H0_RB == H0_RB - 1) ? m / H0_RB : -1)
                                                        : ((m >= H0_RA0 && (m - H0_RA0) % H0_RAS == 0 && (m - H0_RA0) / H0_RAS < MT)
                                                               ? NB + (m - H0_RA0) / H0_RAS
                                                               : -1);
                    if constexpr(rd >= 0)
                        read_one(nst_c, nks, std::integral_constant<int, rd>{}, naf, nbf);
                    if constexpr(SPREAD && !H1 && m == H0_BAR)
                    {
                        // every wave holds the B fragments of both k-steps of this K tile: its B stage may be refilled
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                        __builtin_amdgcn_s_barrier();
                        asm volatile("" ::: "memory");
                    }
                    if constexpr(m % 4 == 3)
                        __builtin_amdgcn_sched_barrier(0);
                });
            };

            // K tile kt, staged in stage ST: k-step 0 out of (af0, bf0) while k-step 1 is read, then k-step 1 while
            // k-step 0 of K tile kt + 1 (stage ST ^ 1) is read and K tile kt + 2 is requested into stage ST.
            auto iteration = [&](auto st, auto other, auto first, auto masked, int kt) {
                const uint32_t k0 = (uint32_t)(kt + 2) * BKB, k_oob = decltype(masked)::value ? k_oob_of(kt + 2) : 0u;
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                half_step(first, std::false_type{}, masked, k0, k_oob, st, af0, bf0, st, std::integral_constant<int, 1>{},
                          af1, bf1);
                // K tile kt is in registers, K tile kt + 1 has landed (the loads of a wave retire in order; with SPREAD
                // the B half of K tile kt + 2 may still be on its way)
                if constexpr(SPREAD)
                    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NLB) : "memory");
                else
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                half_step(std::false_type{}, std::true_type{}, masked, k0, k_oob, st, af1, bf1, other,
                          std::integral_constant<int, 0>{}, af0, bf0);
            };
            using st0 = std::integral_constant<int, 0>;
            using st1 = std::integral_constant<int, 1>;
            // K tile 0, then pairs of iterations whose loads fetch a whole K tile (two copies of the loop body: the
            // stage is a compile-time constant of every address), then the (at most four) whose loads need the mask, with the
            // stage as a scalar
            const int nk_whole = (int)(kbytes / BKB);
            iteration(st0{}, st1{}, std::true_type{}, std::true_type{}, 0);
            int kt = 1;
            for(; kt + 3 < nk_whole; kt += 2)
            {
                iteration(st1{}, st0{}, std::false_type{}, std::false_type{}, kt);
                iteration(st0{}, st1{}, std::false_type{}, std::false_type{}, kt + 1);
            }
            for(; kt < nk - (FUSED ? 0 : 1); ++kt)
                iteration(kt & 1, (kt & 1) ^ 1, std::false_type{}, std::true_type{}, kt);

            // ---- epilogue: 16 consecutive columns of one row per lane, fragment row by fragment row
            const uint32_t lut_lds = smem_lds + (uint32_t)(NST * STAGE);
            // fragment row i through the plain epilogue; G = 0 / 1: one 64-column group of it, G < 0: both
            using both_groups = std::integral_constant<int, -1>;
            auto store_row = [&](auto i_c, auto g_sel) {
                constexpr int i = decltype(i_c)::value, G = decltype(g_sel)::value;
                const int m     = tm * BM + wm * 128 + 16 * i + (lane & 15);
                const int nb    = tn * BN + wn * 128 + 16 * (lane >> 4); // first column of group 0; group 1 is 64 further
                using in_vgpr   = std::integral_constant<bool, (i == MT - 1)>;
                if constexpr(DT == DT_I8 && EPI == EPI_REQUANT_RND)
                {
                    // the values go through the table behind ONE wait per call (both column groups where the caller
                    // allows): with a single wave per SIMD nothing else hides the latency of the byte reads
                    if constexpr(G < 0)
                    {
                        i32x4 v[8];
                        acc_t lo[4], hi[4];
                        fetch_acc(in_vgpr{}, acc[i], 0, lo);
                        fetch_acc(in_vgpr{}, acc[i], 1, hi);
#pragma unroll
                        for(int t = 0; t < 4; ++t)
                            v[t] = lo[t], v[4 + t] = hi[t];
                        int b[32];
                        requant_lut<8>(v, p.scale_gemm, lut_lds, b);
                        if(m < p.M)
                        {
                            int8_t* crow = reinterpret_cast<int8_t*>(c_batch) + (size_t)m * p.ldc;
                            if(nb < p.N)
                                store_bytes16(crow, nb, p.N, vec_ok, b, nt);
                            if(nb + 64 < p.N)
                                store_bytes16(crow, nb + 64, p.N, vec_ok, b + 16, nt);
                        }
                    }
                    else
                    {
                        acc_t v[4];
                        fetch_acc(in_vgpr{}, acc[i], G, v);
                        int b[16];
                        requant_lut<4>(v, p.scale_gemm, lut_lds, b);
                        if(m < p.M && nb + 64 * G < p.N)
                            store_bytes16(reinterpret_cast<int8_t*>(c_batch) + (size_t)m * p.ldc, nb + 64 * G, p.N, vec_ok, b, nt);
                    }
                    return;
                }
#pragma unroll
                for(int g = (G < 0 ? 0 : G); g < (G < 0 ? 2 : G + 1); ++g)
                {
                    if constexpr(DT == DT_I8)
                    {
                        const int n0 = nb + 64 * g;
                        if(m < p.M && n0 < p.N)
                        {
                            acc_t v[4];
                            fetch_acc(in_vgpr{}, acc[i], g, v);
                            int8_t* crow = reinterpret_cast<int8_t*>(c_batch) + (size_t)m * p.ldc;
                            store_row16_i8<EPI>(crow, n0, p.N, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                        }
                    }
                    else
                    {
                        const int n64 = tn * BN + wn * 128 + 64 * g;
                        if(m < p.M && n64 < p.N)
                        {
                            acc_t v[4];
                            fetch_acc(in_vgpr{}, acc[i], g, v);
                            if constexpr(DT == DT_BF16)
                                store_2x8(reinterpret_cast<__bf16*>(c_batch) + (size_t)m * p.ldc, n64, lane >> 4, p.N, vec_ok, v, nt);
                            else
                                store_2x8(reinterpret_cast<_Float16*>(c_batch) + (size_t)m * p.ldc, n64, lane >> 4, p.N, vec_ok, v, nt);
                        }
                    }
                }
            };
            if constexpr(FUSED)
            {
                // the trailing fragment reads and (all-zero) loads; the MFMA results must have left the pipeline before the
                // epilogue reads them (inline-assembly MFMAs are invisible to the compiler's hazard handling)
                asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr(FUSED)
            {
                if(p.epi != EPI_PASSTHROUGH)
                {
                    // A load issued after a store waits for that store too, and this SIMD has no other wave to run
                    // meanwhile: the D values of a whole chunk of fragment rows -- four with one D tensor, two with two (64
                    // registers; eight and four spill) -- are requested before the chunk's first store; a bias row
                    // (stride 0) once per tile. The functor is a compile-time constant of each copy of
                    // the epilogue: a run-time switch per value costs hundreds of scalar branches per tile.
                    const _Float16* d0  = reinterpret_cast<const _Float16*>(p.d0);
                    const _Float16* d1  = reinterpret_cast<const _Float16*>(p.d1);
                    const bool d0_rows  = p.ldd0 != 0;
                    const bool dvec_ok  = ((reinterpret_cast<uintptr_t>(p.d0) | ((uintptr_t)p.ldd0 * ES) |
                                           reinterpret_cast<uintptr_t>(p.d1) | ((uintptr_t)p.ldd1 * ES)) & 15u) == 0;
                    const int q         = lane >> 4;
                    const f16x8 zero8   = {0, 0, 0, 0, 0, 0, 0, 0};
                    auto load8          = [&](const _Float16* row, int n0) {
                        f16x8 x = zero8;
                        if(dvec_ok && n0 + 8 <= p.N)
                            x = *reinterpret_cast<const f16x8*>(row + n0);
                        else
                        {
#pragma unroll
                            for(int e = 0; e < 8; ++e)
                                if(n0 + e < p.N)
                                    x[e] = row[n0 + e];
                        }
                        return x;
                    };
                    auto col0 = [&](int g, int h) { return tn * BN + wn * 128 + 64 * g + 32 * h + 8 * q; };
                    auto with_functor = [&](auto mode_c) {
                        constexpr int MODE    = decltype(mode_c)::value;
                        constexpr bool HAS_D1 = epi_has_d1(MODE);
                        constexpr int CH      = HAS_D1 ? 2 : 4;
                        f16x8 bias[2][2];
#pragma unroll
                        for(int g = 0; g < 2; ++g)
#pragma unroll
                            for(int h = 0; h < 2; ++h)
                                bias[g][h] = (!d0_rows && col0(g, h) < p.N) ? load8(d0, col0(g, h)) : zero8;
                        static_for<MT / CH>([&](auto chunk_c) {
                            constexpr int i0 = decltype(chunk_c)::value * CH;
                            f16x8 x[CH][2][2], y[HAS_D1 ? CH : 1][2][2];
#pragma unroll
                            for(int c = 0; c < CH; ++c)
                            {
                                const int m = tm * BM + wm * 128 + 16 * (i0 + c) + (lane & 15);
#pragma unroll
                                for(int g = 0; g < 2; ++g)
#pragma unroll
                                    for(int h = 0; h < 2; ++h)
                                    {
                                        const bool live = m < p.M && col0(g, h) < p.N;
                                        x[c][g][h] = (live && d0_rows) ? load8(d0 + (size_t)m * p.ldd0, col0(g, h)) : bias[g][h];
                                        if constexpr(HAS_D1)
                                            y[c][g][h] = live ? load8(d1 + (size_t)m * p.ldd1, col0(g, h)) : zero8;
                                    }
                            }
                            static_for<CH>([&](auto c_c) {
                                constexpr int c = decltype(c_c)::value, i = i0 + c;
                                const int m     = tm * BM + wm * 128 + 16 * i + (lane & 15);
#pragma unroll
                                for(int g = 0; g < 2; ++g)
                                {
                                    const int n64 = tn * BN + wn * 128 + 64 * g;
                                    acc_t v[4];
                                    fetch_acc(std::integral_constant<bool, (i == MT - 1)>{}, acc[i], g, v);
#pragma unroll
                                    for(int t = 0; t < 4; ++t)
#pragma unroll
                                        for(int j = 0; j < 4; ++j)
                                        {
                                            const int h = t >> 1, e = 4 * (t & 1) + j;
                                            const float yv = HAS_D1 ? (float)y[HAS_D1 ? c : 0][g][h][e] : 0.0f;
                                            v[t][j] = epi_f16_value<(MODE >= EPI_BILINEAR)>(MODE, v[t][j], (float)x[c][g][h][e], yv,
                                                                                          p.scale_gemm, p.scale_relu);
                                        }
                                    if(m < p.M && n64 < p.N)
                                        store_2x8(reinterpret_cast<_Float16*>(c_batch) + (size_t)m * p.ldc, n64, q, p.N, vec_ok, v, nt);
                                }
                            });
                        });
                    };
                    using std::integral_constant;
                    // (the host sends the functors with a second D tensor to the eight-wave body: their chunks of two
                    // fragment rows serialise four times per tile here -- AddAddFastGelu 125 against 116 us at 4096^3)
                    if(p.epi == EPI_ADD_RELU)
                        with_functor(integral_constant<int, EPI_ADD_RELU>{});
                    else if(p.epi == EPI_CSHUFFLE_ADD_RELU)
                        with_functor(integral_constant<int, EPI_CSHUFFLE_ADD_RELU>{});
                    else
                        with_functor(integral_constant<int, EPI_BILINEAR>{});
                    continue;
                }
            }
            if constexpr(FUSED)
            {
                // (PassThrough on the kernel with the D-operand epilogues)
                static_for<MT>([&](auto i_c) { store_row(i_c, both_groups{}); });
            }
            else
            {
                // ---- the last K tile (in stage kt & 1, its k-step 0 fragments on their way into af0 / bf0) and the
                // epilogue in one: fragment row by fragment row, both k-steps of a row back to back (every accumulator
                // still takes k-step 0 before k-step 1: same sums), so that a row is final 16 MFMAs after the one before
                // it and its conversion and stores run between the MFMAs of the rows behind it. The C tile's way to
                // memory starts seven eighths of a K tile earlier than behind the whole loop. Nothing is loaded and
                // nothing read ahead any more. Rows 0 and 1 take their k-step 0 first, while the k-step 1 fragments
                // arrive.
                const int st = kt & 1;
                auto row_mfmas = [&](auto fi_c, auto ks_c, auto part_c) { // MFMAs 4 * part .. 4 * part + 3 of the row's k-step
                    constexpr int fi = decltype(fi_c)::value, KS = decltype(ks_c)::value;
                    static_for<4>([&](auto j_c) {
                        constexpr int j  = 4 * decltype(part_c)::value + decltype(j_c)::value;
                        constexpr int ft = ((fi + KS) & 1) ? NB - 1 - j : j;
                        if constexpr(KS == 0)
                            mfma<fi == MT - 1, false>(acc[fi][ft], bf0[ft], af0[fi]);
                        else
                            mfma<fi == MT - 1, false>(acc[fi][ft], bf1[ft], af1[fi]);
                    });
                };
                using std::integral_constant;
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                static_for<16>([&](auto m_c) {
                    constexpr int m = decltype(m_c)::value, fi = m / 8, j = m % 8, ft = (fi & 1) ? NB - 1 - j : j;
                    mfma<false, false>(acc[fi][ft], bf0[ft], af0[fi]);
                    read_one(st, integral_constant<int, 1>{}, m_c, af1, bf1); // B fragments 0 .. 7, then A fragments 0 .. 7
                });
                // (LDS reads return in order: all but the last six, the A fragments of rows 2 .. 7)
                asm volatile("s_waitcnt lgkmcnt(6)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                static_for<2>([&](auto fi_c) {
                    row_mfmas(fi_c, integral_constant<int, 1>{}, integral_constant<int, 0>{});
                    row_mfmas(fi_c, integral_constant<int, 1>{}, integral_constant<int, 1>{});
                });
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                // (a row stored here took its last MFMA at least twelve MFMAs ago: the results have left the pipeline;
                // inline-assembly MFMAs are invisible to the compiler's hazard handling)
                static_for<MT - 2>([&](auto r_c) {
                    using fi_c = integral_constant<int, decltype(r_c)::value + 2>;
                    row_mfmas(fi_c{}, integral_constant<int, 0>{}, integral_constant<int, 0>{});
                    __builtin_amdgcn_sched_barrier(0);
                    store_row(r_c, integral_constant<int, 0>{});
                    __builtin_amdgcn_sched_barrier(0);
                    row_mfmas(fi_c{}, integral_constant<int, 0>{}, integral_constant<int, 1>{});
                    row_mfmas(fi_c{}, integral_constant<int, 1>{}, integral_constant<int, 0>{});
                    __builtin_amdgcn_sched_barrier(0);
                    store_row(r_c, integral_constant<int, 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    row_mfmas(fi_c{}, integral_constant<int, 1>{}, integral_constant<int, 1>{});
                });
                asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                store_row(integral_constant<int, MT - 2>{}, both_groups{});
                store_row(integral_constant<int, MT - 1>{}, both_groups{});
            }
        }
    }
};

template <int DT, bool FUSED = false, int EPI = EPI_PASSTHROUGH>
__global__ __launch_bounds__(256) void gemm_w4_kernel(const GemmArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_smem[];
    GemmW4<DT, FUSED, EPI>::run(p, ckx_smem);
}

} // namespace ckx
