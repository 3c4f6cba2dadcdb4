// Weight-streaming GEMM for gfx950: C[M,N] = epilogue(A[M,K] * B[N,K]^T) for 33 .. 128 rows against a large
// weight matrix (LLM linear layers at small token counts), both operands K-contiguous, int8 / fp16 / bf16.
//
// Such a problem is bound by reading B out of HBM exactly once, and what decides the rate is how many bytes of B
// every CU keeps in flight -- with both operands staged through LDS (the tile kernel) that is one or two stages of
// a tile. Here B never touches LDS: a wave owns 16 * NTW output columns and loads its B fragments straight from
// global memory into registers in MFMA operand layout (lane l: row l % 16, 16 bytes at k-step offset 16 * (l / 16)),
// D K tiles ahead of their use -- no other wave needs them. Only A (at most 128 rows, L2 resident) is shared by the
// four waves of a workgroup and goes through an LDS ring of D + 1 stages, filled by direct global->LDS loads with the
// XOR-swizzled chunk order of the tile kernel. All loads of a wave retire in order, so one counted
// s_waitcnt vmcnt((D - 1) * loads-per-tile) says that K tile k has landed, A and B alike; one barrier per K tile.
//
// A work unit is (block of 64 * NTW columns, K run): when the column blocks alone cannot cover the chip the K
// extent is cut into runs whose raw accumulators go to the caller's workspace ([run][M][N] int32 / fp32, the layout
// of the tile kernel's K split) and splitk_reduce_kernel adds them in run order and applies the epilogue.
//
// Purpose of DeviceGemmSplitK in the reference (include/ck/tensor_operation/gpu/device/device_gemm_splitk.hpp:14-39):
// fill the machine when M x N has few tiles; the kernel body replaces kernel_gemm_xdl_cshuffle_v1.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

template <int DT, int MT, int NTW, int D>
struct GemmStream
{
    static constexpr int NW     = 4;
    static constexpr int NT     = NW * 64;
    static constexpr int ES     = DT == DT_I8 ? 1 : 2;
    static constexpr int BM     = MT * 16;
    static constexpr int BN     = NW * NTW * 16;
    static constexpr int A_TILE = BM * 128;      // bytes of an A stage: BM rows x 128 bytes of K
    static constexpr int NSTA   = D + 1;
    static constexpr int LDS    = NSTA * A_TILE;
    static constexpr int NLA    = BM * 8 / NT;   // 16-byte direct loads per thread and K tile (A)
    static constexpr int NLB    = NTW * 2;       // 16-byte register loads per thread and K tile (B: two k-steps)
    static constexpr int LPT    = NLA + NLB;
    static_assert(MT % 2 == 0 && MT >= 2, "an A stage is a whole number of 256-thread load rounds");
    static_assert(D >= 2 && (D - 1) * LPT < 64, "vmcnt is a 6-bit counter");

    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;

    __device__ static __forceinline__ void run(const GemmArgs& p, uint8_t* smem)
    {
        const int tid  = threadIdx.x;
        const int lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t frow = (uint32_t)(lane & 15), fq = (uint32_t)(lane >> 4);

        const int nblocks = p.tiles_n;                   // column blocks of BN
        const int unit    = (int)blockIdx.x;
        const int sp      = unit / nblocks;              // K run
        const int n0      = (unit - sp * nblocks) * BN;
        const uint32_t kbytes = (uint32_t)p.K * ES;
        const int nk_real = (int)((kbytes + 127) / 128);
        const int nk      = nk_real > 0 ? nk_real : 1;
        const int k_begin = sp * p.nk_per;
        const int k_end   = k_begin + p.nk_per < nk ? k_begin + p.nk_per : nk;

        const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a, p.a_bytes);
        const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b, p.b_bytes);

        // ---- A: slot j of this thread fills LDS row (j * NW + wave) * 8 + lane / 8, chunk position lane % 8, with
        // global chunk (lane % 8) ^ (row & 7) of that row
        const uint32_t kb = ((uint32_t)(lane & 7) ^ (uint32_t)((lane >> 3) & 7)) << 4;
        uint32_t a_off[NLA];
#pragma unroll
        for(int j = 0; j < NLA; ++j)
        {
            const uint32_t r = (uint32_t)((j * NW + wave) * 8 + (lane >> 3));
            a_off[j]         = r < (uint32_t)p.M ? r * (uint32_t)p.lda * ES + kb : kOutOfRange;
        }
        // ---- B: fragment t of this wave, MFMA row i = lane % 16, holds column 4 * NTW * (i / 4) + 4 * t + i % 4 of
        // the wave's 16 * NTW, so that after D^T = B_frag x A_frag a lane owns 4 * NTW CONSECUTIVE columns
        uint32_t b_off[NTW];
#pragma unroll
        for(int t = 0; t < NTW; ++t)
        {
            const uint32_t n = (uint32_t)n0 + (uint32_t)(wave * NTW * 16) + 4u * NTW * (frow >> 2) + 4u * t + (frow & 3u);
            b_off[t]         = n < (uint32_t)p.N ? n * (uint32_t)p.ldb * ES + fq * 16 : kOutOfRange;
        }

        acc_t acc[MT][NTW];
#pragma unroll
        for(int i = 0; i < MT; ++i)
#pragma unroll
            for(int t = 0; t < NTW; ++t)
                acc[i][t] = acc_t{0, 0, 0, 0};

        i32x4 bq[NSTA][NLB]; // B fragments of the K tiles in flight, [slot][2 * t + k-step]

        // loads of K tile kt into slot s: A (direct to LDS) first, then B (registers). K tiles past the run and
        // chunks past K use an out-of-range offset: zeros arrive and the count of loads in flight stays the same.
        auto issue_tile = [&](int kt, auto slot_c) {
            constexpr int S   = decltype(slot_c)::value;
            const uint32_t k0 = (uint32_t)kt * 128u;
            const bool live   = kt < k_end;
            const uint32_t a_oob = (live && k0 + kb < kbytes) ? 0u : kOutOfRange;
#pragma unroll
            for(int j = 0; j < NLA; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(smem + S * A_TILE + (j * NW + wave) * 1024), 16,
                                                         (a_off[j] + k0) | a_oob, 0, 0, 0);
#pragma unroll
            for(int t = 0; t < NTW; ++t)
#pragma unroll
                for(int ks = 0; ks < 2; ++ks)
                {
                    const uint32_t kk = k0 + (uint32_t)ks * 64u;
                    const uint32_t o  = (live && kk + fq * 16 < kbytes) ? 0u : kOutOfRange;
                    bq[S][2 * t + ks] =
                        __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, (b_off[t] + kk) | o, 0, 0));
                }
        };

        const uint32_t smem_lds = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
        // A fragment i of k-step ks: row 16 i + lane % 16, chunk 4 ks + lane / 16 at position chunk ^ (row & 7)
        const uint32_t fa0 = frow * 128u + (((0u + fq) ^ (frow & 7u)) << 4);
        const uint32_t fa1 = frow * 128u + (((4u + fq) ^ (frow & 7u)) << 4);

        auto mfma = [&](acc_t& c, const i32x4& b, const i32x4& a) {
            if constexpr(DT == DT_I8)
                c = __builtin_amdgcn_mfma_i32_16x16x64_i8(b, a, c, 0, 0, 0);
            else if constexpr(DT == DT_BF16)
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b), __builtin_bit_cast(bf16x8, a), c, 0, 0, 0);
            else
                c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, b), __builtin_bit_cast(f16x8, a), c, 0, 0, 0);
        };

        // ---- prologue: D K tiles in flight
        static_for<D>([&](auto s_c) { issue_tile(k_begin + decltype(s_c)::value, s_c); });

        // One K tile: slot S = (kt - k_begin) % NSTA, a compile-time constant in the unrolled bodies below.
        auto tile_step = [&](int kt, auto s_c) {
            constexpr int S = decltype(s_c)::value;
            // K tile kt has landed once at most the D - 1 tiles requested after it are outstanding
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 1) * LPT) : "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // every wave is past its reads of tile kt - 1: its stage and its B registers take tile kt + D
            issue_tile(kt + D, std::integral_constant<int, (S + D) % NSTA>{});
            __builtin_amdgcn_sched_barrier(0);

            const uint32_t st = smem_lds + (uint32_t)(S * A_TILE);
            i32x4 af0[MT], af1[MT];
            static_for<MT>([&](auto i_c) {
                af0[decltype(i_c)::value] = lds_read_b128<decltype(i_c)::value * 16 * 128>(st + fa0);
            });
            static_for<MT>([&](auto i_c) {
                af1[decltype(i_c)::value] = lds_read_b128<decltype(i_c)::value * 16 * 128>(st + fa1);
            });
            // (reads the compiler does not know about: waited for by hand; the first k-step's fragments were
            // issued first and LDS reads return in order)
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(MT) : "memory");
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for(int t = 0; t < NTW; ++t)
#pragma unroll
                for(int i = 0; i < MT; ++i)
                    mfma(acc[i][t], bq[S][2 * t], af0[i]);
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for(int t = 0; t < NTW; ++t)
#pragma unroll
                for(int i = 0; i < MT; ++i)
                    mfma(acc[i][t], bq[S][2 * t + 1], af1[i]);
            __builtin_amdgcn_sched_barrier(0);
        };
        // Whole groups of NSTA K tiles run without a condition inside the loop body: with one, the compiler can no
        // longer count the loads between a B fragment's request and its use across the back edge and waits for
        // (nearly) all of them. The last, partial group is straight-line code after the loop.
        const int n_tiles = k_end - k_begin;
        const int k_full  = k_begin + n_tiles / NSTA * NSTA;
        for(int kt0 = k_begin; kt0 < k_full; kt0 += NSTA)
            static_for<NSTA>([&](auto s_c) { tile_step(kt0 + decltype(s_c)::value, s_c); });
        static_for<NSTA - 1>([&](auto s_c) {
            if(k_full + decltype(s_c)::value < k_end) // (uniform over the workgroup)
                tile_step(k_full + decltype(s_c)::value, s_c);
        });
        // the trailing (all-zero) direct loads still target LDS
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

        // ---- epilogue: lane owns row 16 i + lane % 16, columns n0 + wave * 16 NTW + 4 NTW * (lane / 16) + 4 t + j
        constexpr int CW = 4 * NTW; // consecutive columns of a lane
        const int nn     = n0 + wave * NTW * 16 + CW * (int)fq;
#pragma unroll
        for(int i = 0; i < MT; ++i)
        {
            const int m = 16 * i + (int)frow;
            if(m >= p.M || nn >= p.N)
                continue;
            if(p.ksplit > 1)
            {
                uint8_t* wrow = reinterpret_cast<uint8_t*>(p.ws) + (((size_t)sp * p.M + m) * p.N + nn) * 4;
                if(nn + CW <= p.N && (p.N & 3) == 0)
                {
#pragma unroll
                    for(int t = 0; t < NTW; ++t)
                        reinterpret_cast<acc_t*>(wrow)[t] = acc[i][t];
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < CW; ++e)
                        if(nn + e < p.N)
                            reinterpret_cast<decltype(acc[0][0][0] + 0)*>(wrow)[e] = acc[i][e / 4][e % 4];
                }
            }
            else if constexpr(DT == DT_I8)
            {
                int b[CW];
#pragma unroll
                for(int e = 0; e < CW; ++e)
                {
                    const int v = acc[i][e / 4][e % 4];
                    b[e]        = p.epi == EPI_REQUANT_RND  ? requant_rnd(v, p.scale_gemm, p.scale_relu)
                                  : p.epi == EPI_REQUANT_CK ? requant_ck(v, p.scale_gemm, p.scale_relu)
                                                            : v;
                }
                int8_t* crow = reinterpret_cast<int8_t*>(p.c) + (size_t)m * p.ldc + nn;
                if(nn + CW <= p.N && (reinterpret_cast<uintptr_t>(crow) & (CW - 1)) == 0)
                {
                    int pk[NTW];
#pragma unroll
                    for(int t = 0; t < NTW; ++t)
                        pk[t] = pack4_low_bytes(b[4 * t], b[4 * t + 1], b[4 * t + 2], b[4 * t + 3]);
                    if constexpr(NTW == 1)
                        *reinterpret_cast<int*>(crow) = pk[0];
                    else
                        *reinterpret_cast<i32x2*>(crow) = i32x2{pk[0], pk[1]};
                }
                else
                {
#pragma unroll
                    for(int e = 0; e < CW; ++e)
                        if(nn + e < p.N)
                            crow[e] = (int8_t)b[e];
                }
            }
            else
            {
                using T = typename std::conditional<DT == DT_BF16, __bf16, _Float16>::type;
                T* crow = reinterpret_cast<T*>(p.c) + (size_t)m * p.ldc + nn;
#pragma unroll
                for(int e = 0; e < CW; ++e)
                    if(nn + e < p.N)
                        crow[e] = (T)acc[i][e / 4][e % 4];
            }
        }
    }
};

template <int DT, int MT, int NTW, int D>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const GemmArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_stream_smem[];
    GemmStream<DT, MT, NTW, D>::run(p, ckx_stream_smem);
}

// Stream instances: rows covered, columns per workgroup. launch_stream(dt, which, ...) launches instance `which`
// on a grid of (column blocks x K runs) workgroups; GemmArgs::tiles_n = column blocks, ksplit / nk_per / ws as for the
// tile kernel's K split (the caller runs splitk_reduce_kernel afterwards when ksplit > 1).
struct StreamInstance
{
    const char* name;
    int max_m, bn;
};
extern const StreamInstance kStreamInstances[];
extern const int kNumStreamInstances;
hipError_t launch_stream(int dt, int which, const GemmArgs& a, hipStream_t s);

} // namespace ckx
