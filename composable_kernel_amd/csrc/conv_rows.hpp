// 1x1 convolution forward for gfx950 with a SHORT pixel (64 or 128 bytes: 64 int8 / fp16 channels, 128 int8 channels; with
// 64 or 128 output channels also 256 bytes, with 64 also 512) and at most 256 output channels per workgroup column: out[M, K] = epilogue(in[M, C] * wei[K, C]^T), M = N * Ho * Wo,
// stride 1, no padding (the input IS the [M, C] matrix).
//
// Such layers move 100 - 500 MB through 4 - 16 KB of weights: pure streaming. On the tile kernel every 256-row tile is one
// K iteration -- load, wait, multiply, store -- with one tile of prefetch per workgroup, and an int8 layer, which has half
// the bytes of its fp16 twin in flight, runs no faster than it. Here nothing goes through LDS and nothing waits at a
// barrier: a wave keeps ALL weights of its column block in registers as MFMA operands (K / 16 fragments per k-step),
// loads 16 rows at a time straight into the other operand's layout (lane l: row l % 16, 16 bytes at 16 * (l / 16) of the
// k-step: for a 64-byte pixel one instruction fetches 1 KB of consecutive memory), and stores every finished row as 16
// consecutive outputs per lane. Products are issued as D^T = W_frag x pixel_frag with the weight rows of a 64-column group
// permuted (b_row_to_col), so that lane (m = l % 16, q = l / 16) ends up with columns 16 q .. 16 q + 15 of row m -- the
// ownership the tile kernel's row stores are written for. Two row tiles per iteration, the next two in flight.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct ConvRowsArgs
{
    const void* in;
    const void* wei;
    void* out;
    const void* bias; // fp16 [K] (FUSED: bias + ReLU)
    uint32_t in_bytes;
    int M, C, Kout;
    int epi;
    float scale_gemm, scale_relu;
    int nt_store;
};

// KS k-steps per pixel (pixel = 64 * KS bytes), NG 64-column groups per workgroup column (block of 64 * NG output channels)
template <int DT, int KS, int NG, bool FUSED>
__global__ __launch_bounds__(256) void conv_rows_kernel(const ConvRowsArgs p)
{
    using acc_t      = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    constexpr int ES = DT == DT_I8 ? 1 : 2;
    constexpr int U  = KS >= 8 ? 1 : 2; // row tiles per iteration (a 512-byte pixel's row tile is 32 registers already)
    const int lane   = threadIdx.x & 63;
    const int wave   = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t r = lane & 15, q = lane >> 4;
    const int kblock = blockIdx.y * 64 * NG; // first output channel of this workgroup's column block

    const __amdgpu_buffer_rsrc_t rsrc_in  = make_rsrc(p.in, p.in_bytes);
    const __amdgpu_buffer_rsrc_t rsrc_wei = make_rsrc(p.wei, (uint32_t)p.Kout * (uint32_t)p.C * ES);

    // ---- weights: fragment (g, t, ks) holds, in lane (j = l % 16, q), 16 bytes of weight row 64 g + b_row_to_col(16 t + j)
    i32x4 w[NG][4][KS];
#pragma unroll
    for(int g = 0; g < NG; ++g)
#pragma unroll
        for(int t = 0; t < 4; ++t)
        {
            const uint32_t k = (uint32_t)kblock + 64u * g + b_row_to_col(16u * t + r);
#pragma unroll
            for(int ks = 0; ks < KS; ++ks)
                w[g][t][ks] = __builtin_bit_cast(
                    i32x4, __builtin_amdgcn_raw_buffer_load_b128(
                               rsrc_wei, k < (uint32_t)p.Kout ? k * (uint32_t)(64 * KS) + 64u * ks + 16u * q : kOutOfRange, 0, 0));
        }
    f16x8 b_lo[FUSED ? NG : 1], b_hi[FUSED ? NG : 1];
    if constexpr(FUSED)
    {
#pragma unroll
        for(int g = 0; g < NG; ++g)
        {
            // (K comes in whole groups of 64: a group past K -- K = 192 in a block of 256 -- has no bias to read)
            const _Float16* b = reinterpret_cast<const _Float16*>(p.bias) + kblock + 64 * g + 16 * q;
            const f16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
            const bool live   = kblock + 64 * g < p.Kout;
            b_lo[g]           = live ? *reinterpret_cast<const f16x8*>(b) : zero8;
            b_hi[g]           = live ? *reinterpret_cast<const f16x8*>(b + 8) : zero8;
        }
    }

    // ---- row tiles: the waves of the launch take them in turn, U at a time (all waves read one stretch of memory)
    const int nwaves  = (int)gridDim.x * 4;
    const int gwave   = (int)blockIdx.x * 4 + wave;
    const int ntiles  = (p.M + 15) / 16;
    const int ngroups = (ntiles + U - 1) / U;
    auto load_rows = [&](int grp, i32x4(&a)[U][KS]) {
#pragma unroll
        for(int u = 0; u < U; ++u)
        {
            const uint32_t m = (uint32_t)(grp * U + u) * 16u + r;
#pragma unroll
            for(int ks = 0; ks < KS; ++ks)
                a[u][ks] = __builtin_bit_cast(
                    i32x4, __builtin_amdgcn_raw_buffer_load_b128(
                               rsrc_in, m < (uint32_t)p.M ? m * (uint32_t)(64 * KS) + 64u * ks + 16u * q : kOutOfRange, 0, 0));
        }
    };
    const bool vec_ok = ((reinterpret_cast<uintptr_t>(p.out) | ((uintptr_t)p.Kout * ES)) & 15u) == 0;
    const bool nt     = p.nt_store != 0;
    auto finish_rows  = [&](int grp, const i32x4(&a)[U][KS]) {
#pragma unroll
        for(int u = 0; u < U; ++u)
        {
            const int m = (grp * U + u) * 16 + (int)r;
#pragma unroll
            for(int g = 0; g < NG; ++g)
            {
                acc_t acc[4];
#pragma unroll
                for(int t = 0; t < 4; ++t)
                {
#pragma unroll
                    for(int ks = 0; ks < KS; ++ks)
                    {
                        const acc_t c = ks == 0 ? acc_t{0, 0, 0, 0} : acc[t];
                        if constexpr(DT == DT_I8)
                            acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[g][t][ks], a[u][ks], c, 0, 0, 0);
                        else
                            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w[g][t][ks]),
                                                                         __builtin_bit_cast(f16x8, a[u][ks]), c, 0, 0, 0);
                    }
                }
                const int n0 = kblock + 64 * g + 16 * (int)q;
                if(m < p.M && n0 < p.Kout)
                {
                    if constexpr(DT == DT_I8)
                    {
                        int8_t* crow      = reinterpret_cast<int8_t*>(p.out) + (size_t)m * p.Kout;
                        const i32x4 v[4] = {acc[0], acc[1], acc[2], acc[3]};
                        if(p.epi == EPI_REQUANT_RND)
                            store_row16_i8<EPI_REQUANT_RND>(crow, n0, p.Kout, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                        else if(p.epi == EPI_REQUANT_CK)
                            store_row16_i8<EPI_REQUANT_CK>(crow, n0, p.Kout, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                        else
                            store_row16_i8<EPI_PASSTHROUGH>(crow, n0, p.Kout, vec_ok, v, p.scale_gemm, p.scale_relu, nt);
                    }
                    else
                    {
                        _Float16* crow = reinterpret_cast<_Float16*>(p.out) + (size_t)m * p.Kout;
                        f32x4 v[4]     = {acc[0], acc[1], acc[2], acc[3]};
                        if constexpr(FUSED)
                        {
#pragma unroll
                            for(int t = 0; t < 4; ++t)
#pragma unroll
                                for(int j = 0; j < 4; ++j)
                                {
                                    const int e = 4 * t + j;
                                    v[t][j] = epi_f16_value<false>(EPI_ADD_RELU, v[t][j], (float)(e < 8 ? b_lo[g][e & 7] : b_hi[g][e & 7]), 0.0f);
                                }
                        }
                        store_row16_f16(crow, n0, p.Kout, vec_ok, v, nt);
                    }
                }
            }
        }
    };

    i32x4 a0[U][KS], a1[U][KS];
    int grp = gwave;
    if(grp < ngroups)
        load_rows(grp, a0);
    while(grp < ngroups)
    {
        // (past the last group the offsets are out of range: the loads return zeros and nothing is stored)
        load_rows(grp + nwaves, a1);
        finish_rows(grp, a0);
        grp += nwaves;
        if(grp >= ngroups)
            break;
        load_rows(grp + nwaves, a0);
        finish_rows(grp, a1);
        grp += nwaves;
    }
}

// pixel_bytes 64 or 128 with Kout a multiple of 64 (above 256: of 256), 256 with Kout 64 / 128, 512 with Kout 64; fused: fp16 bias + ReLU
hipError_t launch_conv_rows(int dt, int pixel_bytes, bool fused, const ConvRowsArgs& a, hipStream_t s);

} // namespace ckx
