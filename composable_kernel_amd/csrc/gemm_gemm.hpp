// Batched fused GEMM-GEMM for gfx950, fp16:  C[g] = half( half(A[g] * B0[g]) * B1[g] ).
// A [G,M,K] row-major, B0 stored [G,N,K] (column-major K x N), B1 [G,N,O] row-major,
// C [G,M,O] row-major (layout gmk_gnk_gno_gmo of upstream's DeviceBatchedGemmGemm; batch
// offsets as in kernel_batched_gemm_xdlops_v2r3, device_batched_gemm_xdl.hpp:79-88).
//
// One workgroup owns 64 or 128 rows of one batch and walks N in steps of 128 columns; the next
// step's B0 / B1 slices are prefetched into registers while the current one is multiplied.
// The slice of the intermediate never leaves registers:
//   gemm0 is issued as S^T = B0_frag x A_frag, so lane (l%16 = m, l/16 = q) holds S[m][n]
//   for 4 values of n per MFMA tile; the B0 rows fed to a PAIR of tiles are chosen so that
//   the pair gives the lane n = 32*pair + 8q .. +7, i.e. exactly the eight K-slots that the
//   same lane must supply as the second operand of gemm1 (C^T = B1T_frag x S_frag) after a
//   round-to-nearest-even conversion to fp16. B1 is transposed while it is staged into LDS
//   so that its fragment is one 16-byte read as well.
//
// SOFTMAX variant (upstream's DeviceBatchedGemmSoftmaxGemm, "attention"):
//   C[g] = half( half(softmax_n(scale * A[g] * B0[g], masked)) * B1[g] )
// with the softmax along N in one pass over N (running row maximum and running sum): a step's
// scores become p = exp(s - running max), the output accumulators and the running sum are rescaled
// whenever the maximum grows, and the division by the sum happens once at the end. A row's 128
// scores of a step sit in four lanes (l%16 = row, l/16 = q), 32 each: the row maximum crosses those
// lanes with v_permlane16_swap / v_permlane32_swap, and so does the final sum. Columns past N and, with the
// upper-triangle mask, columns n > m count as -infinity; masked-out steps are skipped altogether.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <string>

#include "gemm_tile.hpp"

namespace ckx {

struct GemmGemmArgs
{
    const _Float16* a;
    const _Float16* b0;
    const _Float16* b1;
    _Float16* c;
    int M, N, K, O, batch;
    int sa, sb0, sb1, sc;
    int64_t bsa, bsb0, bsb1, bsc;
    int slabs; // ceil(M / rows per workgroup)
    float scale;   // softmax variant: scores are scale * (A * B0)
    int mask_upper; // softmax variant: scores with n > m are masked out
};

// maximum / sum over the four lanes l, l^16, l^32, l^48 (every one of them gets the result)
typedef short s16x4_t __attribute__((__vector_size__(4 * sizeof(short))));
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4;

__device__ __forceinline__ float quad_rows_sum(float x)
{
    auto a = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, x), false, false);
    const uint32_t a0 = a[0], a1 = a[1];
    x      = __builtin_bit_cast(float, a0) + __builtin_bit_cast(float, a1);
    auto b = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, x), false, false);
    const uint32_t b0 = b[0], b1 = b[1];
    return __builtin_bit_cast(float, b0) + __builtin_bit_cast(float, b1);
}
// Maxima of scores as bare v_max_f32 / v_max3_f32. In front of every fmaxf operand that it cannot prove to be a quiet
// number (an MFMA result, a lane swap) the compiler puts a canonicalising v_max_f32 x, x, x, which doubled the
// instructions of the running maximum. (A NaN score makes its row of the output NaN through the exponentials
// whatever the maximum is.) The compiler does not see what an asm statement reads, so it cannot keep the distance
// that the hardware asks for between an MFMA and a VALU read of its result: mfma_results_settle() goes between.
__device__ __forceinline__ float max2_valu(float a, float b)
{
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float max3_valu(float a, float b, float c)
{
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
// 24 wait states after the MFMAs issued so far, and nothing scheduled across: more than the longest
// MFMA-write-to-VALU-read distance of the architecture (passes + 3 wait states for the 16-pass instructions).
__device__ __forceinline__ void mfma_results_settle()
{
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 7");
    __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ float quad_rows_max(float x)
{
    auto a = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, x), false, false);
    const uint32_t a0 = a[0], a1 = a[1];
    x      = max2_valu(__builtin_bit_cast(float, a0), __builtin_bit_cast(float, a1));
    auto b = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, x), false, false);
    const uint32_t b0 = b[0], b1 = b[1];
    return max2_valu(__builtin_bit_cast(float, b0), __builtin_bit_cast(float, b1));
}

// KS  k-steps of gemm0 (K padded to 32*KS), OG  64-column groups of the output (O padded to 64*OG),
// MT  16-row MFMA tiles per wave, NW waves: a workgroup owns 16*MT*NW rows of one batch.
template <int KS, int OG, int MT, int NW>
struct GemmGemmCfg
{
    static constexpr int NT   = 64 * NW;
    static constexpr int BM   = 16 * MT * NW;
    static constexpr int BNC  = 128; // columns of the intermediate per step
    static constexpr int KP   = KS * 32;
    static constexpr int OP   = OG * 64;
    // LDS rows are unpadded and their 16-byte chunks XOR-swizzled with bits of the row index (ab_key / b1_key).
    // A ds_read_b128 is served in four cycles of 16 lanes each, and the lanes of a cycle are those with equal
    // (lane bit 5, parity of lane bits 2..4) -- measured with random bank-balanced address patterns, which that
    // partition predicts exactly; row padding (16 bytes) left every fragment read of this kernel with two- to
    // four-way bank conflicts under it (SQ_LDS_BANK_CONFLICT = half of SQ_LDS_IDX_ACTIVE). The keys make the 16
    // lanes of every cycle of every fragment read land on 16 different 16-byte bank groups.
    static constexpr int AST  = KP * 2; // LDS row stride of A / B0 (bytes)
    // chunk position of chunk c of staged row r of A / B0: c ^ ab_key(r)
    __device__ static __forceinline__ uint32_t ab_key(uint32_t r)
    {
        // (KP / 8 chunks per row: 4, 8 or 16 -- the key stays inside the row)
        return (((r >> 3) & 1u) << 1) | (KP >= 64 ? ((r >> 1) & 1u) << 2 : 0u) | (KP == 128 ? (r & 1u) << 3 : 0u);
    }
    // The B1 slice of a step stays as it is in memory, [n][o] (row stride B1RS bytes), and the gemm1 operand -- for
    // one o, eight consecutive n -- comes out of it through the transposing read ds_read_b64_tr_b16: within 16 lanes,
    // lane 4e + j points at four consecutive o of row n + e, and lane i receives element i of the 16 so addressed
    // in each of the four rows. (Transposing on the way in took 32 two-byte LDS writes per thread and step.)
    // b1_key(n): XOR mask on the byte offset inside row n, so that the 32 lanes of a half wave (rows n + e and
    // n + 8 + e, four 8-byte pieces each) touch 32 different 8-byte bank pairs: with 128-byte rows the parity of n
    // already selects the bank half and bits 1 and 3 of n move the piece (bits 3, 4 of the offset); 256-byte rows
    // all start at bank 0, and bit 0 of n swaps the two 128-byte halves as well.
    static constexpr int B1RS = OP * 2;
    __device__ static __forceinline__ uint32_t b1_key(uint32_t n)
    {
        return (((n >> 1) & 1u) << 3) | (((n >> 3) & 1u) << 4) | (OG == 2 ? (n & 1u) << 7 : 0u);
    }
    static constexpr int A_BYTES   = BM * AST;
    static constexpr int B0_BYTES  = BNC * AST;
    static constexpr int B1T_BYTES = BNC * B1RS;
    static constexpr int LDS       = A_BYTES + B0_BYTES + B1T_BYTES;
    static constexpr int KCH = KP / 8; // 16-byte chunks per staged row of A / B0
    static constexpr int OCH = OP / 8;
    static constexpr int NB0 = BNC * KCH / NT; // 16-byte loads per thread and step
    static constexpr int NB1 = BNC * OCH / NT;
    static_assert(NB0 >= 1 && NB1 >= 1, "too many threads for one step");
};

template <int KS, int OG, int MT, int NW, bool SOFTMAX = false>
// (the 32-row-per-wave softmax variant for small K and O is held to 256 registers, two waves per SIMD: one
// wave's exponentials then overlap the other's MFMAs; left alone the compiler takes 340 and runs one)
__global__ __launch_bounds__(NW * 64)
    __attribute__((amdgpu_waves_per_eu(SOFTMAX && MT == 2 && KS <= 2 && OG == 1 ? 2 : 1))) void gemm_gemm_kernel(
        const GemmGemmArgs p)
{
    using Cfg = GemmGemmCfg<KS, OG, MT, NW>;
    constexpr int KCH = Cfg::KCH, OCH = Cfg::OCH, NB0 = Cfg::NB0, NB1 = Cfg::NB1, NT = Cfg::NT;
    extern __shared__ __attribute__((aligned(16))) uint8_t gg_smem[];
    uint8_t* sA   = gg_smem;
    uint8_t* sB0  = sA + Cfg::A_BYTES;
    uint8_t* sB1T = sB0 + Cfg::B0_BYTES;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int fr   = lane & 15; // MFMA row/col index supplied by this lane
    const int q    = lane >> 4; // K-slot group

    // Workgroups of one batch share B0[g] and B1[g]: keep them on one XCD (ids are dealt
    // round-robin over 8 XCDs) so that those panels are fetched into one L2 only.
    int g, slab;
    {
        const int nb = p.slabs * p.batch;
        const int bid = blockIdx.x;
        if((p.batch & 7) == 0)
        {
            const int xcd = bid & 7, local = bid >> 3;
            g    = xcd + 8 * (local / p.slabs);
            slab = local - (local / p.slabs) * p.slabs;
        }
        else
        {
            g    = bid / p.slabs;
            slab = bid - g * p.slabs;
        }
        (void)nb;
    }
    const int m0       = slab * Cfg::BM;
    const _Float16* A  = p.a + (int64_t)g * p.bsa;
    const _Float16* B0 = p.b0 + (int64_t)g * p.bsb0;
    const _Float16* B1 = p.b1 + (int64_t)g * p.bsb1;
    _Float16* C        = p.c + (int64_t)g * p.bsc;
    const i32x4 zero4  = {0, 0, 0, 0};

    // ---- register prefetch of one step's B0 / B1 slices ------------------------------------
    // Buffer loads: one resource per operand over the batch's rows, and per thread and load a byte offset that is fixed
    // for the whole kernel (row inside the slice, 16-byte chunk; out of range for chunks past K / O) -- a step adds its
    // first row, one addition per load, and rows past N read as zeros through the range check.
    const __amdgpu_buffer_rsrc_t rsrc_b0 = make_rsrc(B0, p.N > 0 ? (uint32_t)(((int64_t)(p.N - 1) * p.sb0 + p.K) * 2) : 0u);
    const __amdgpu_buffer_rsrc_t rsrc_b1 = make_rsrc(B1, p.N > 0 ? (uint32_t)(((int64_t)(p.N - 1) * p.sb1 + p.O) * 2) : 0u);
    uint32_t vb0[NB0], vb1[NB1];
#pragma unroll
    for(int i = 0; i < NB0; ++i)
    {
        const int idx = tid + NT * i;
        const int row = idx / KCH, ch = idx - row * KCH;
        vb0[i]        = ch * 8 < p.K ? (uint32_t)row * (uint32_t)p.sb0 * 2u + (uint32_t)ch * 16u : kOutOfRange;
    }
#pragma unroll
    for(int i = 0; i < NB1; ++i)
    {
        const int idx = tid + NT * i;
        const int row = idx / OCH, ch = idx - row * OCH;
        vb1[i]        = ch * 8 < p.O ? (uint32_t)row * (uint32_t)p.sb1 * 2u + (uint32_t)ch * 16u : kOutOfRange;
    }
    i32x4 rb0[NB0], rb1[NB1];
    auto load_into = [&](int n0, i32x4(&r0)[NB0], i32x4(&r1)[NB1]) {
        const uint32_t step0 = (uint32_t)n0 * (uint32_t)p.sb0 * 2u, step1 = (uint32_t)n0 * (uint32_t)p.sb1 * 2u;
#pragma unroll
        for(int i = 0; i < NB0; ++i)
            r0[i] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b0, vb0[i] + step0, 0, 0));
#pragma unroll
        for(int i = 0; i < NB1; ++i)
            r1[i] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b1, vb1[i] + step1, 0, 0));
    };
    auto load_step = [&](int n0) { load_into(n0, rb0, rb1); };
    auto store_step = [&]() {
#pragma unroll
        for(int i = 0; i < NB0; ++i)
        {
            const int idx = tid + NT * i;
            const int row = idx / KCH, ch = idx - row * KCH;
            *reinterpret_cast<i32x4*>(sB0 + row * Cfg::AST + ((uint32_t)ch ^ Cfg::ab_key((uint32_t)row)) * 16) = rb0[i];
        }
#pragma unroll
        for(int i = 0; i < NB1; ++i)
        {
            const int idx = tid + NT * i;
            const int row = idx / OCH, ch = idx - row * OCH;
            // (two 8-byte halves: the key may swap them)
            uint8_t* dst = sB1T + row * Cfg::B1RS;
            const uint32_t off = (uint32_t)(ch * 16) ^ Cfg::b1_key((uint32_t)row);
            *reinterpret_cast<i32x2*>(dst + off)       = i32x2{rb1[i][0], rb1[i][1]};
            *reinterpret_cast<i32x2*>(dst + (off ^ 8)) = i32x2{rb1[i][2], rb1[i][3]};
        }
    };

    // the same for the second register set of the two-step prefetch (unused, and gone, where PF == 1)
    i32x4 rb0b[NB0], rb1b[NB1];
    auto store_from = [&](const i32x4(&r0)[NB0], const i32x4(&r1)[NB1]) {
#pragma unroll
        for(int i = 0; i < NB0; ++i)
        {
            const int idx = tid + NT * i;
            const int row = idx / KCH, ch = idx - row * KCH;
            *reinterpret_cast<i32x4*>(sB0 + row * Cfg::AST + ((uint32_t)ch ^ Cfg::ab_key((uint32_t)row)) * 16) = r0[i];
        }
#pragma unroll
        for(int i = 0; i < NB1; ++i)
        {
            const int idx = tid + NT * i;
            const int row = idx / OCH, ch = idx - row * OCH;
            uint8_t* dst = sB1T + row * Cfg::B1RS;
            const uint32_t off = (uint32_t)(ch * 16) ^ Cfg::b1_key((uint32_t)row);
            *reinterpret_cast<i32x2*>(dst + off)       = i32x2{r1[i][0], r1[i][1]};
            *reinterpret_cast<i32x2*>(dst + (off ^ 8)) = i32x2{r1[i][2], r1[i][3]};
        }
    };

    load_step(0);

    // ---- A slab -> LDS -> registers (kept for the whole kernel) -----------------------
    for(int idx = tid; idx < Cfg::BM * KCH; idx += NT)
    {
        const int row = idx / KCH, ch = idx - row * KCH;
        const int m = m0 + row, k = ch * 8;
        i32x4 v = zero4;
        if(m < p.M && k < p.K)
            v = *reinterpret_cast<const i32x4*>(A + (int64_t)m * p.sa + k);
        *reinterpret_cast<i32x4*>(sA + row * Cfg::AST + ((uint32_t)ch ^ Cfg::ab_key((uint32_t)row)) * 16) = v;
    }
    __syncthreads();
    f16x8 af[MT][KS];
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
#pragma unroll
        for(int ks = 0; ks < KS; ++ks)
        {
            const uint32_t arow = (uint32_t)(wave * 16 * MT + mt * 16 + fr);
            af[mt][ks] = *reinterpret_cast<const f16x8*>(sA + arow * Cfg::AST + ((uint32_t)(ks * 4 + q) ^ Cfg::ab_key(arow)) * 16);
        }

    // byte offset inside the B1 slice that this lane addresses in the transposing reads of gemm1
    const uint32_t b1_lane =
        (uint32_t)(8 * q + (fr >> 2)) * Cfg::B1RS + ((uint32_t)(32 * (fr & 3)) ^ Cfg::b1_key((uint32_t)(8 * q + (fr >> 2))));

    f32x4 acc1[MT][OG * 4];
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
#pragma unroll
        for(int t = 0; t < OG * 4; ++t)
            acc1[mt][t] = f32x4{0, 0, 0, 0};

    // softmax state of the MT rows this lane holds scores of (identical in the four lanes of a row,
    // except row_sum, which is each lane's share until the end)
    constexpr float kLog2e = 1.4426950408889634f;
    const float ninf       = -__builtin_inff();
    float row_max[MT], row_sum[MT];
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
        row_max[mt] = ninf, row_sum[mt] = 0.0f;
    // (never exactly 0: a masked score is -inf, and -inf * 0 would be a NaN; with the smallest normal number
    // instead, scale 0 still turns every unmasked score into 0)
    const float c2 = __builtin_fmaxf(__builtin_fabsf(p.scale) * kLog2e, 1.17549435e-38f);
    if(SOFTMAX && p.scale < 0.0f)
    {
        // scores = scale * (A * B0) = |scale| * ((-A) * B0): flip the sign bits of the A fragments once
#pragma unroll
        for(int mt = 0; mt < MT; ++mt)
#pragma unroll
            for(int ks = 0; ks < KS; ++ks)
                af[mt][ks] = __builtin_bit_cast(f16x8, __builtin_bit_cast(i32x4, af[mt][ks]) ^ (int)0x80008000);
    }
    // with the upper-triangle mask, columns past the slab's last row are masked for every row of it
    const int n_end = (SOFTMAX && p.mask_upper && m0 + Cfg::BM < p.N) ? m0 + Cfg::BM : p.N;

    // ---- main loop over the steps ---------------------------------------------------------------------------
    // A step's MFMAs take well under a microsecond, a load out of HBM longer: with one step of register prefetch
    // every step of a short problem (N = 512: four steps) ends waiting for its successor's slices. Where the
    // registers allow, the slices of TWO steps are in flight (PF == 2: a second register set, the loop unrolled by
    // two). The softmax variants and the largest plain one have no room (they would spill) and keep one.
    constexpr int PF = ((MT == 2 && NW == 4) || (SOFTMAX && (NW != 8 || (KS == 4 && OG == 2)))) ? 1 : 2;
    if constexpr(PF == 1)
    {
        for(int n0 = 0; n0 < n_end; n0 += Cfg::BNC)
        {
            __syncthreads(); // everyone is done reading the previous step from LDS
            store_step();
            __syncthreads();
            if(n0 + Cfg::BNC < n_end)
                load_step(n0 + Cfg::BNC); // in flight while this step is multiplied
#include "gemm_gemm_step.inc"
        }
    }
    else
    {
        // step i lives in register set i % 2 until it goes to LDS
        if(Cfg::BNC < n_end)
            load_into(Cfg::BNC, rb0b, rb1b);
        for(int nb = 0; nb < n_end; nb += 2 * Cfg::BNC)
        {
            {
                const int n0 = nb;
                __syncthreads();
                store_from(rb0, rb1);
                __syncthreads();
                if(n0 + 2 * Cfg::BNC < n_end)
                    load_into(n0 + 2 * Cfg::BNC, rb0, rb1);
#include "gemm_gemm_step.inc"
            }
            if(nb + Cfg::BNC < n_end)
            {
                const int n0 = nb + Cfg::BNC;
                __syncthreads();
                store_from(rb0b, rb1b);
                __syncthreads();
                if(n0 + 2 * Cfg::BNC < n_end)
                    load_into(n0 + 2 * Cfg::BNC, rb0b, rb1b);
#include "gemm_gemm_step.inc"
            }
        }
    }

    const bool vec_ok = ((reinterpret_cast<uintptr_t>(C) | ((uintptr_t)p.sc * 2)) & 15u) == 0;
    if constexpr(SOFTMAX)
    {
#pragma unroll
        for(int mt = 0; mt < MT; ++mt)
        {
            const float total = quad_rows_sum(row_sum[mt]);
            const float inv   = total > 0.0f ? 1.0f / total : 0.0f; // N == 0: an empty sum, C = 0
#pragma unroll
            for(int ot = 0; ot < OG * 4; ++ot)
                acc1[mt][ot] = acc1[mt][ot] * inv;
        }
    }
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
    {
        const int m = m0 + wave * 16 * MT + mt * 16 + fr;
        if(m >= p.M)
            continue;
#pragma unroll
        for(int og = 0; og < OG; ++og)
        {
            const int o0 = 64 * og + 16 * q;
            if(o0 >= p.O)
                continue;
            const f32x4 v[4] = {acc1[mt][og * 4], acc1[mt][og * 4 + 1], acc1[mt][og * 4 + 2],
                                acc1[mt][og * 4 + 3]};
            store_row16_f16(C + (int64_t)m * p.sc, o0, p.O, vec_ok, v);
        }
    }
}

// ---------------------------------------------------------------- host side
constexpr int kNumGemmGemmInstances = 3;

inline const char* gemm_gemm_instance_name(int i)
{
    return i == 0   ? "MI355X_Mfma16_GemmGemm<128 rows, 4 waves x 32, 128-col steps, K<=128, O<=128>"
           : i == 1 ? "MI355X_Mfma16_GemmGemm<64 rows, 4 waves x 16, 128-col steps, K<=128, O<=128>"
                    : "MI355X_Mfma16_GemmGemm<128 rows, 8 waves x 16, 128-col steps, K<=128, O<=128>";
}

inline bool gemm_gemm_supported(int M, int N, int K, int O, int batch, int sa, int sb0, int sb1, int sc,
                                int64_t bsa, int64_t bsb0, int64_t bsb1, int64_t bsc, int instance,
                                std::string& why)
{
    (void)bsc;
    if(M < 0 || N < 0 || K < 0 || O < 0 || batch < 0)
        return why = "invalid: negative dimension", false;
    if(instance < -1 || instance >= kNumGemmGemmInstances)
        return why = "invalid: no such instance", false;
    if(K > 128 || O > 128)
        return why = "K and O above 128 are not built", false;
    if(K % 8 || O % 8 || sa % 8 || sb0 % 8 || sb1 % 8 || bsa % 8 || bsb0 % 8 || bsb1 % 8)
        return why = "K, O and the A/B0/B1 strides must be multiples of 8 elements (16 bytes)", false;
    if(sa < K || sb0 < K || sb1 < O || sc < O)
        return why = "stride smaller than the contiguous extent", false;
    if((long)((M + 63) / 64) * batch >= (1l << 31))
        return why = "grid too large", false;
    // (the slices of a batch are addressed through 32-bit buffer offsets)
    if((long)N * sb0 * 2 >= (1l << 31) || (long)N * sb1 * 2 >= (1l << 31))
        return why = "B0 / B1 of one batch must stay below 2 GiB", false;
    return true;
}

template <int KS, int OG, int MT, int NW, bool SOFTMAX>
inline hipError_t gemm_gemm_launch_t(GemmGemmArgs a, hipStream_t s)
{
    using Cfg  = GemmGemmCfg<KS, OG, MT, NW>;
    auto* kern = &gemm_gemm_kernel<KS, OG, MT, NW, SOFTMAX>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    a.slabs = (a.M + Cfg::BM - 1) / Cfg::BM;
    hipLaunchKernelGGL(kern, dim3(a.slabs * a.batch), dim3(Cfg::NT), Cfg::LDS, s, a);
    return hipGetLastError();
}

template <int MT, int NW, bool SOFTMAX>
inline hipError_t gemm_gemm_launch_mt(const GemmGemmArgs& g, hipStream_t s)
{
    const int ks = g.K <= 32 ? 1 : (g.K <= 64 ? 2 : 4);
    const int og = g.O <= 64 ? 1 : 2;
    if(ks == 1)
        return og == 1 ? gemm_gemm_launch_t<1, 1, MT, NW, SOFTMAX>(g, s) : gemm_gemm_launch_t<1, 2, MT, NW, SOFTMAX>(g, s);
    if(ks == 2)
        return og == 1 ? gemm_gemm_launch_t<2, 1, MT, NW, SOFTMAX>(g, s) : gemm_gemm_launch_t<2, 2, MT, NW, SOFTMAX>(g, s);
    return og == 1 ? gemm_gemm_launch_t<4, 1, MT, NW, SOFTMAX>(g, s) : gemm_gemm_launch_t<4, 2, MT, NW, SOFTMAX>(g, s);
}

// softmax: the attention variant with scores scale * (A * B0) and the optional upper-triangle mask
inline hipError_t gemm_gemm_launch(const void* a, const void* b0, const void* b1, void* c, int M, int N, int K,
                                   int O, int batch, int sa, int sb0, int sb1, int sc, int64_t bsa,
                                   int64_t bsb0, int64_t bsb1, int64_t bsc, int instance, hipStream_t s,
                                   bool softmax = false, float scale = 1.0f, bool mask_upper = false)
{
    GemmGemmArgs g;
    g.a = (const _Float16*)a, g.b0 = (const _Float16*)b0, g.b1 = (const _Float16*)b1, g.c = (_Float16*)c;
    g.M = M, g.N = N, g.K = K, g.O = O, g.batch = batch;
    g.sa = sa, g.sb0 = sb0, g.sb1 = sb1, g.sc = sc;
    g.bsa = bsa, g.bsb0 = bsb0, g.bsb1 = bsb1, g.bsc = bsc;
    g.slabs = 0;
    g.scale = scale, g.mask_upper = mask_upper;
    if(instance < 0)
    {
        // Many short waves (8 x 16 rows, the instance with two steps of prefetch where registers allow) are ahead on
        // short problems: G 64, 512 x 64 x 512 x 64 plain 8.5 against 10.1 us, with softmax 10.9 against 13.0. Over a
        // long N with small heads the 32-row waves read the B0 / B1 fragments half as often per row and win: G 64,
        // 4096 x 64 x 4096 x 64 plain 267 against 302 us, softmax 367 against 433 (2048: 76 / 85 and 102 / 115; at
        // N = 1024 plain 23.5 / 26.2, softmax 31.3 / 34.0).
        // That needs workgroups to spare (two of them share a CU): below 256 slabs of 128 rows the 8-wave instance
        // stays ahead with softmax (G 8, 2048 x 64 x 2048 x 64: 30.1 against 37.2 us), and without it, up to 128
        // slabs of small heads, the 64-row instance, which doubles the workgroups (20.6 against 25.4 us).
        const long slabs128 = (long)batch * ((M + 127) / 128);
        const bool small_heads = K <= 64 && O <= 64;
        instance = (!softmax && small_heads && slabs128 <= 128) ? 1 : (small_heads && N >= 1024 && slabs128 >= 256) ? 0 : 2;
    }
    if(softmax)
        return instance == 0 ? gemm_gemm_launch_mt<2, 4, true>(g, s)
               : instance == 1 ? gemm_gemm_launch_mt<1, 4, true>(g, s)
                               : gemm_gemm_launch_mt<1, 8, true>(g, s);
    return instance == 0 ? gemm_gemm_launch_mt<2, 4, false>(g, s)
           : instance == 1 ? gemm_gemm_launch_mt<1, 4, false>(g, s)
                           : gemm_gemm_launch_mt<1, 8, false>(g, s);
}

} // namespace ckx
