// Skinny GEMM for gfx950: C[M,N] = epilogue(A[M,K] * B[N,K]^T) with M <= 16*MT (a few token
// rows against a large weight matrix), int8 or fp16, same layouts as the tile kernel.
//
// Such problems are bound by streaming B out of HBM exactly once. Each workgroup owns 16*NT
// output columns (NT > 1: every A fragment, which comes out of L2, is used NT times) and the
// WHOLE K extent, split over its waves: a wave loads its K slice of
// the 16 B rows straight from global memory into registers in the MFMA operand layout (lane
// l: row l%16, 16 bytes at k-step offset 16*(l/16)) -- there is no reuse across waves, so
// there is no LDS staging -- multiplies it with the matching A fragments (read through L2),
// and the per-wave partial tiles are summed through LDS at the end. No split-K workspace, no
// atomics, and thousands of independent 1 KB loads in flight per CU.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

// Epilogue and store of one lane's four consecutive outputs (row m, columns nn .. nn + 3) of a summed 16 x 16
// accumulator tile in the D^T = B_frag x A_frag lane layout: lane (m % 16, q) holds columns 4q .. 4q + 3.
template <int DT, typename ACC>
__device__ __forceinline__ void store_quad(const GemmArgs& p, const ACC& s, int m, int nn)
{
    // lane (m = lane%16, q): columns 4q .. 4q+3 of the tile's 16, row 16*mt + m
    if(m >= p.M || nn >= p.N)
        return;
    if constexpr(DT == DT_I8)
    {
        int b[4];
        if(epi_per_column_scale(p.epi))
        {
            const float* sc = reinterpret_cast<const float*>(p.d0);
#pragma unroll
            for(int j = 0; j < 4; ++j)
                b[j] = nn + j < p.N ? mul2_clamp(s[j], sc[nn + j], p.epi == EPI_RELU_MUL2_CLAMP) : 0;
        }
        else
        {
#pragma unroll
            for(int j = 0; j < 4; ++j)
                b[j] = p.epi == EPI_REQUANT_RND  ? requant_rnd(s[j], p.scale_gemm, p.scale_relu)
                       : p.epi == EPI_REQUANT_CK ? requant_ck(s[j], p.scale_gemm, p.scale_relu)
                                                 : s[j];
        }
        int8_t* crow = reinterpret_cast<int8_t*>(p.c) + (size_t)m * p.ldc + nn;
        if(nn + 4 <= p.N && ((reinterpret_cast<uintptr_t>(crow)) & 3u) == 0)
            *reinterpret_cast<int*>(crow) = pack4_low_bytes(b[0], b[1], b[2], b[3]);
        else
        {
#pragma unroll
            for(int j = 0; j < 4; ++j)
                if(nn + j < p.N)
                    crow[j] = (int8_t)b[j];
        }
    }
    else if constexpr(DT == DT_BF16)
    {
        __bf16* crow = reinterpret_cast<__bf16*>(p.c) + (size_t)m * p.ldc + nn;
#pragma unroll
        for(int j = 0; j < 4; ++j)
            if(nn + j < p.N)
                crow[j] = (__bf16)s[j];
    }
    else
    {
        _Float16* crow       = reinterpret_cast<_Float16*>(p.c) + (size_t)m * p.ldc + nn;
        const _Float16* d0row = reinterpret_cast<const _Float16*>(p.d0) + (size_t)m * p.ldd0 + nn;
        const _Float16* d1row = reinterpret_cast<const _Float16*>(p.d1) + (size_t)m * p.ldd1 + nn;
#pragma unroll
        for(int j = 0; j < 4; ++j)
            if(nn + j < p.N)
            {
                float val = s[j];
                if(p.epi != EPI_PASSTHROUGH)
                    val = epi_f16_value(p.epi, val, (float)d0row[j], epi_has_d1(p.epi) ? (float)d1row[j] : 0.0f,
                                        p.scale_gemm, p.scale_relu);
                crow[j] = (_Float16)val;
            }
    }
}

template <int DT, int MT, int NW, int KU, int NT = 1>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const GemmArgs p)
{
    using acc_t = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    constexpr int ES = DT == DT_I8 ? 1 : 2;
    __shared__ acc_t red[NW][MT][NT][64];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * 16 * NT;

    const uint32_t kbytes = (uint32_t)p.K * ES;
    const int ksteps      = (int)((kbytes + 63u) >> 6);
    const int per_wave    = (ksteps + NW - 1) / NW;
    const int ks_begin    = wave * per_wave;
    const int ks_end      = ks_begin + per_wave < ksteps ? ks_begin + per_wave : ksteps;

    const __amdgpu_buffer_rsrc_t rsrc_a = make_rsrc(p.a, p.a_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_b = make_rsrc(p.b, p.b_bytes);

    uint32_t b_off[NT];
#pragma unroll
    for(int nt = 0; nt < NT; ++nt)
    {
        const uint32_t n = (uint32_t)n0 + 16u * nt + r;
        b_off[nt]        = n < (uint32_t)p.N ? n * (uint32_t)p.ldb * ES + q * 16 : kOutOfRange;
    }
    uint32_t a_off[MT];
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
        a_off[mt] = 16u * mt + r < (uint32_t)p.M ? (16u * mt + r) * (uint32_t)p.lda * ES + q * 16 : kOutOfRange;

    acc_t acc[MT][NT];
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
#pragma unroll
        for(int nt = 0; nt < NT; ++nt)
            acc[mt][nt] = acc_t{0, 0, 0, 0};

    // one chunk = KU consecutive k-steps (64 bytes of K each); k-steps at or past ks_end and the
    // K tail read as zeros through an out-of-range buffer offset
    auto load_chunk = [&](int ks0, i32x4(&bq)[NT][KU], i32x4(&aq)[MT][KU]) {
#pragma unroll
        for(int u = 0; u < KU; ++u)
        {
            const int ks        = ks0 + u;
            const uint32_t kb   = (uint32_t)ks * 64u;
            const bool ok       = ks < ks_end && kb + q * 16 < kbytes;
#pragma unroll
            for(int nt = 0; nt < NT; ++nt)
                bq[nt][u] = __builtin_bit_cast(
                    i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, ok ? b_off[nt] + kb : kOutOfRange, 0, 0));
#pragma unroll
            for(int mt = 0; mt < MT; ++mt)
                aq[mt][u] = __builtin_bit_cast(
                    i32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, ok ? a_off[mt] + kb : kOutOfRange, 0, 0));
        }
    };
    auto mfma_chunk = [&](const i32x4(&bq)[NT][KU], const i32x4(&aq)[MT][KU]) {
#pragma unroll
        for(int u = 0; u < KU; ++u)
#pragma unroll
            for(int mt = 0; mt < MT; ++mt)
#pragma unroll
                for(int nt = 0; nt < NT; ++nt)
                {
                    if constexpr(DT == DT_I8)
                        acc[mt][nt] =
                            __builtin_amdgcn_mfma_i32_16x16x64_i8(bq[nt][u], aq[mt][u], acc[mt][nt], 0, 0, 0);
                    else if constexpr(DT == DT_BF16)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, bq[nt][u]), __builtin_bit_cast(bf16x8, aq[mt][u]), acc[mt][nt],
                            0, 0, 0);
                    else
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            __builtin_bit_cast(f16x8, bq[nt][u]), __builtin_bit_cast(f16x8, aq[mt][u]), acc[mt][nt],
                            0, 0, 0);
                }
    };

    i32x4 b0[NT][KU], a0[MT][KU], b1[NT][KU], a1[MT][KU];
    load_chunk(ks_begin, b0, a0);
    for(int ks = ks_begin; ks < ks_end; ks += 2 * KU)
    {
        load_chunk(ks + KU, b1, a1);
        mfma_chunk(b0, a0);
        load_chunk(ks + 2 * KU, b0, a0);
        mfma_chunk(b1, a1);
    }

    // ---- sum the waves' partial tiles, then the epilogue on wave 0 ---------------------
#pragma unroll
    for(int mt = 0; mt < MT; ++mt)
#pragma unroll
        for(int nt = 0; nt < NT; ++nt)
            red[wave][mt][nt][lane] = acc[mt][nt];
    __syncthreads();
    // the (mt, nt) accumulator tiles are dealt round-robin to the waves for the final sum
#pragma unroll
    for(int t = 0; t < MT * NT; ++t)
    {
        if(t % NW != wave)
            continue;
        const int mt = t / NT, nt = t % NT;
        acc_t s = red[0][mt][nt][lane];
#pragma unroll
        for(int w = 1; w < NW; ++w)
        {
            const acc_t v = red[w][mt][nt][lane];
            s[0] += v[0], s[1] += v[1], s[2] += v[2], s[3] += v[3];
        }
        // lane (m = lane%16, q): columns 4q .. 4q+3 of the tile's 16, row 16*mt + m
        store_quad<DT>(p, s, 16 * mt + (int)r, n0 + 16 * nt + 4 * (int)q);
    }
}

} // namespace ckx
