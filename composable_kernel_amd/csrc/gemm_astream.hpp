// Weight-streaming GEMM for a few dozen to 128 rows (LLM prefill of a short prompt against a large weight matrix):
// C[M,N] = epilogue(A[M,K] * B[N,K]^T), M <= 16 * MT, A row-major, B column-major, both K-contiguous.
//
// B (the weights) must come out of HBM exactly once and is the only stream that has to run at HBM speed; A is small, sits
// in L2, and every workgroup needs all of it -- at 128 rows, 2.7 bytes of A for every byte of B. The loads of ONE WAVE
// return in order: an L2-hit load issued behind an HBM-latency load of the same wave waits for it (measured with a
// two-wave probe: a wave streaming an L2-resident region with eight 1 KB loads in flight takes 64 ns per load alone, 78 ns
// while ANOTHER wave of the CU streams HBM misses with sixteen in flight, and 327 ns when it interleaves one miss per hit
// itself). A wave that loads both operands therefore pays an HBM round trip for every burst of A. Here the two streams
// belong to different waves:
//   * a workgroup owns 16 * NT output columns and the whole K extent, cut into 128-byte K tiles that are dealt to four
//     PAIRS of waves in turn (pair w: K tiles w, w + 4, ...); the pairs never wait for each other's data;
//   * the pair's LOADER wave (waves 4 .. 7, one per SIMD) requests the pair's next A tile -- all rows x 128 bytes, 16 KB --
//     into one of the pair's two LDS slots by direct loads and waits for it: L2 hits only, never behind a miss;
//   * the pair's COMPUTE wave (waves 0 .. 3) requests its B fragments straight into registers in MFMA operand layout,
//     RB - 1 steps ahead (a ring of RB register sets: two microseconds of HBM latency), reads the A fragments of the
//     current slot with ds_read_b128 (XOR-swizzled chunks, as in the tile kernel) and issues the MFMAs;
//   * one workgroup barrier per step hands the slots over; the compute waves' partial tiles are added through LDS at the
//     end (fixed order), the epilogue runs on the sums;
//   * every workgroup walks K from a different starting K tile (see `rot`): they all read the same A, and an L2 channel
//     serves identical requests one at a time.
// No K split across workgroups, no workspace, one launch.
#pragma once

#include "gemm_skinny.hpp"

namespace ckx {

template <int DT, int MT, int NT, int RB = 4>
struct GemmAStream
{
    static constexpr int NP = 4, NTHR = 2 * NP * 64; // pairs; compute waves 0 .. NP - 1, loader waves NP .. 2 NP - 1
    static constexpr int ES   = DT == DT_I8 ? 1 : 2;
    static constexpr int ROWS = MT * 16;
    static constexpr int SLOT = ROWS * 128;       // one K tile of A: all rows x 128 bytes
    static constexpr int PAIR_LDS = 2 * SLOT;
    static constexpr int LDS      = NP * PAIR_LDS;
    static constexpr int NLA = ROWS / 8;          // direct loads (1 KB each) of an A tile
    static constexpr int NLB = NT * 2;            // register loads of the B fragments of a K tile (two k-steps)
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    static_assert(RB % 2 == 0 && RB >= 2, "the LDS slot of a step is a compile-time constant of the unrolled loop");
    static_assert(MT * NT * 1024 * NP <= LDS, "the compute waves' partial tiles are summed through LDS");

    __device__ static __forceinline__ void run(const GemmArgs& p, uint8_t* smem)
    {
        const int lane = threadIdx.x & 63;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const bool loader = wave >= NP;
        const int pair    = loader ? wave - NP : wave;
        const uint32_t r = lane & 15, q = lane >> 4;
        const int n0 = blockIdx.x * 16 * NT;

        const uint32_t kbytes = (uint32_t)p.K * ES;
        const int ktiles      = (int)((kbytes + 127) / 128);
        int nsteps            = (ktiles + NP - 1) / NP;   // steps of a pair
        nsteps                = (nsteps + RB - 1) / RB * RB; // (whole turns of the register ring; steps past the end see zeros)
        // Every workgroup needs all of A. Walking K in the same order, all of them would ask the L2 for the same lines at
        // the same moment, and an L2 channel serves one of them at a time (measured: 256 workgroups streaming the same
        // 512 KB in the same order get 54 GB/s each, 116 GB/s when each starts at its own offset): workgroup b starts at K
        // tile rot and wraps. Pair w takes the K tiles (NP * step + w + rot) mod ktiles, in the order of its steps.
        const int rot = ktiles > 0 ? (int)((blockIdx.x * 13u) % (unsigned)ktiles) : 0;
        // byte offset into K of the pair's K tile of a step, or past the end (zeros) for the steps that pad the ring
        auto tile_kb = [&](int step) {
            const int li = step * NP + pair;
            const int kt = li + rot < ktiles ? li + rot : li + rot - ktiles;
            return li < ktiles ? (uint32_t)kt * 128u : 0xfffffff0u;
        };

        uint8_t* const pair_lds = smem + pair * PAIR_LDS;
        acc_t acc[MT][NT];
#pragma unroll
        for(int i = 0; i < MT; ++i)
#pragma unroll
            for(int t = 0; t < NT; ++t)
                acc[i][t] = acc_t{0, 0, 0, 0};

        if(loader)
        {
            // A tile: load slot g deposits rows 8 g .. 8 g + 7 x 128 bytes; a lane fills chunk position lane % 8 of row
            // 8 g + lane / 8 with chunk (lane % 8) ^ (row & 7) of that row
            const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a, p.a_bytes);
            const uint32_t a_chunk = ((uint32_t)(lane & 7) ^ (uint32_t)(lane >> 3)) << 4;
            uint32_t a_off[NLA];
#pragma unroll
            for(int g = 0; g < NLA; ++g)
            {
                const uint32_t row = 8u * g + (uint32_t)(lane >> 3);
                a_off[g]           = row < (uint32_t)p.M ? row * (uint32_t)p.lda * ES + a_chunk : kOutOfRange;
            }
            auto load_a = [&](int step) {
                const uint32_t kb = tile_kb(step);
                const bool ok     = kb < kbytes && kb + a_chunk < kbytes;
                uint8_t* const slot = pair_lds + (step & 1) * SLOT;
#pragma unroll
                for(int g = 0; g < NLA; ++g)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(slot + g * 1024), 16,
                                                             ok ? a_off[g] + kb : kOutOfRange, 0, 0, 0);
            };
            load_a(0);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            for(int s = 0; s < nsteps; ++s)
            {
                // the slot of step s + 1 was read in step s - 1, which ended with a barrier
                load_a(s + 1);
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
            }
        }
        else
        {
            const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b, p.b_bytes);
            // B fragment of N tile t: lane (r, q) holds 16 bytes of row n0 + 16 t + r at k-step offset 16 q
            uint32_t b_off[NT];
#pragma unroll
            for(int t = 0; t < NT; ++t)
            {
                const uint32_t n = (uint32_t)n0 + 16u * t + r;
                b_off[t]         = n < (uint32_t)p.N ? n * (uint32_t)p.ldb * ES + q * 16 : kOutOfRange;
            }
            // fragment (i, ks) of a slot: row 16 i + r, chunk 4 ks + q
            const uint32_t pair_lds_a = (uint32_t)(uintptr_t)(lds_ptr_t)pair_lds;
            const uint32_t fr[2] = {pair_lds_a + r * 128u + (((0u + q) ^ (r & 7u)) << 4),
                                    pair_lds_a + r * 128u + (((4u + q) ^ (r & 7u)) << 4)};
            auto load_b = [&](int step, i32x4(&bq)[NT][2]) {
                const uint32_t kb = tile_kb(step);
#pragma unroll
                for(int ks = 0; ks < 2; ++ks)
                {
                    const bool ok = kb < kbytes && kb + ks * 64 + q * 16 < kbytes;
#pragma unroll
                    for(int t = 0; t < NT; ++t)
                        bq[t][ks] = __builtin_bit_cast(
                            i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, ok ? b_off[t] + kb + ks * 64 : kOutOfRange, 0, 0));
                }
            };
            // one step: per k-step MT fragment reads (inline assembly, waited for here) and MT x NT MFMAs
            auto compute = [&](auto slot_c, const i32x4(&bq)[NT][2]) {
                constexpr int SL = decltype(slot_c)::value;

                static_for<2>([&](auto ks_c) {
                    constexpr int ks = decltype(ks_c)::value;
                    i32x4 af[MT];
                    static_for<MT>([&](auto i_c) {
                        constexpr int i = decltype(i_c)::value;
                        af[i]           = lds_read_b128<SL * SLOT + i * 2048>(fr[ks]);
                    });
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for(int i = 0; i < MT; ++i)
#pragma unroll
                        for(int t = 0; t < NT; ++t)
                        {
                            if constexpr(DT == DT_I8)
                                acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bq[t][ks], af[i], acc[i][t], 0, 0, 0);
                            else if constexpr(DT == DT_BF16)
                                acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                    __builtin_bit_cast(bf16x8, bq[t][ks]), __builtin_bit_cast(bf16x8, af[i]), acc[i][t], 0, 0, 0);
                            else
                                acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    __builtin_bit_cast(f16x8, bq[t][ks]), __builtin_bit_cast(f16x8, af[i]), acc[i][t], 0, 0, 0);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                });
            };
            i32x4 bq[RB][NT][2];
            static_for<RB - 1>([&](auto j_c) { load_b(decltype(j_c)::value, bq[decltype(j_c)::value]); });
            __builtin_amdgcn_s_barrier(); // (the loader's first A tile has landed)
            for(int s0 = 0; s0 < nsteps; s0 += RB)
            {
                static_for<RB>([&](auto j_c) {
                    constexpr int j = decltype(j_c)::value;
                    load_b(s0 + j + RB - 1, bq[(j + RB - 1) % RB]);
                    compute(std::integral_constant<int, j % 2>{}, bq[j]);
                    // this step's slot may be refilled, the next step's A tile has landed
                    __builtin_amdgcn_s_barrier();
                });
            }
        }
        // trailing (all-zero) loads
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);

        // ---- sum the compute waves' partial tiles through LDS, in wave order, then the epilogue: tile (i, t) on wave
        // (i * NT + t) % (2 NP) -- the loader waves take their share of it
        if(!loader)
        {
            acc_t* const red = reinterpret_cast<acc_t*>(smem) + wave * (MT * NT * 64);
#pragma unroll
            for(int i = 0; i < MT; ++i)
#pragma unroll
                for(int t = 0; t < NT; ++t)
                    red[(i * NT + t) * 64 + lane] = acc[i][t];
        }
        __syncthreads();
#pragma unroll
        for(int x = 0; x < MT * NT; ++x)
        {
            if(x % (2 * NP) != wave)
                continue;
            const int i = x / NT, t = x % NT;
            const acc_t* const red = reinterpret_cast<const acc_t*>(smem);
            acc_t s = red[x * 64 + lane];
#pragma unroll
            for(int w = 1; w < NP; ++w)
            {
                const acc_t v = red[w * (MT * NT * 64) + x * 64 + lane];
                s[0] += v[0], s[1] += v[1], s[2] += v[2], s[3] += v[3];
            }
            store_quad<DT>(p, s, 16 * i + (int)r, n0 + 16 * t + 4 * (int)q);
        }
    }
};

template <int DT, int MT, int NT, int RB = 4>
__global__ __launch_bounds__(512) void gemm_astream_kernel(const GemmArgs p)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t ckx_smem[];
    GemmAStream<DT, MT, NT, RB>::run(p, ckx_smem);
}

} // namespace ckx
