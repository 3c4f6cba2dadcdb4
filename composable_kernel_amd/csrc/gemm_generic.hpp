// Element-granular GEMM / implicit-GEMM conv forward for gfx950: the instance that takes what the vectorised
// instances refuse -- a K (or, for a K-major operand, an M / N) extent, a leading dimension, a channel count
// or a base address that is not a whole 16-byte vector.
//
// Takes the place of the reference's padded GEMM instances (GemmSpecialization::KPadding / MNKPadding,
// include/ck/tensor_operation/gpu/device/gemm_specialization.hpp:10-20, device_gemm_xdl_cshuffle.hpp:99-184)
// and of its odd-channel conv instances (ConvolutionForwardSpecialization::OddC,
// convolution_forward_specialization.hpp:13-19; device test case C = 3, test/convnd_fwd/conv2d_fwd.cpp:111),
// which load with SrcScalarPerVector = 1. As there, the price is bandwidth: every operand element is its own
// load instruction unless a whole 16-byte chunk happens to be in range, contiguous and aligned.
//
// One workgroup of 4 waves (2 x 2) computes a 64 x 64 tile of C; a K tile is ONE MFMA k-step (64 int8 /
// 32 fp16 or bf16 values = 64 bytes of every row). Thread t gathers 16 bytes of row t / 4 of the A tile and of
// the B tile into registers -- zeros where the row, the K index or the conv window is out of range, which is the
// whole of "padding" -- and writes them to LDS (rows padded to 80 bytes); after a barrier every wave reads two A and
// two B fragments and issues four MFMAs (D^T = B_frag x A_frag, so a lane owns 4 consecutive columns of one row).
// Operand layouts are run-time element strides, so all four GEMM layouts, a strided batch and the 1-D / 2-D / 3-D
// im2col view go through the same code. Epilogues: PassThrough, both requant forms (int8), the add / ReLU functors
// with D operands (fp16), applied per element.
#pragma once

#include "gemm_tile.hpp"

namespace ckx {

struct GenericLayout
{
    long a_sm, a_sk; // element strides of A(m, k)
    long b_sn, b_sk; // element strides of B(k, n)
    int X, Y;        // filter extents of the two innermost spatial dimensions (im2col only)
};

template <int DT, int IM2COL>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const GemmArgs p, const GenericLayout lay)
{
    constexpr int ES    = DT == DT_I8 ? 1 : 2;
    constexpr int EPC   = 16 / ES;  // elements of a 16-byte chunk
    constexpr int KT    = 4 * EPC;  // K elements per tile: one MFMA k-step
    constexpr int PITCH = 80;       // LDS bytes per staged row
    using elem_t = typename std::conditional<DT == DT_I8, uint8_t, uint16_t>::type;
    using acc_t  = typename std::conditional<DT == DT_I8, i32x4, f32x4>::type;
    __shared__ __attribute__((aligned(16))) uint8_t sa[64 * PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t sb[64 * PITCH];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int tm = (int)(blockIdx.x % (unsigned)p.tiles_m), tn = (int)(blockIdx.x / (unsigned)p.tiles_m);
    const long g = blockIdx.y;

    const elem_t* A = reinterpret_cast<const elem_t*>(p.a) + g * p.bsa;
    const elem_t* B = reinterpret_cast<const elem_t*>(p.b) + g * p.bsb;

    // this thread's slot of both staged tiles: row lrow, 16-byte chunk lchunk
    const int lrow = tid >> 2, lchunk = tid & 3;
    const long gm = (long)tm * 64 + lrow, gn = (long)tn * 64 + lrow;
    const bool m_ok = gm < p.M, n_ok = gn < p.N;

    // im2col: window origin of output pixel gm (device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:224-301 in closed form)
    long img = 0;
    int hi0 = 0, wi0 = 0, d0 = 0;
    if constexpr(IM2COL != 0)
    {
        if(m_ok)
        {
            uint32_t rem = (uint32_t)gm, n;
            if constexpr(IM2COL == 2)
            {
                n                 = magic_div(rem, p.cv.div_dhowo);
                const uint32_t r3 = rem - n * p.cv.div_dhowo.d;
                const uint32_t od = magic_div(r3, p.cv.div_howo);
                rem               = r3 - od * p.cv.div_howo.d;
                d0                = (int)od * p.cv.sD - p.cv.pF;
            }
            else
            {
                n   = magic_div(rem, p.cv.div_howo);
                rem = rem - n * p.cv.div_howo.d;
            }
            const uint32_t ho = magic_div(rem, p.cv.div_wo);
            const uint32_t wo = rem - ho * p.cv.div_wo.d;
            hi0               = (int)ho * p.cv.sH - p.cv.pT;
            wi0               = (int)wo * p.cv.sW - p.cv.pL;
            img               = n;
        }
    }

    acc_t acc[2][2];
#pragma unroll
    for(int i = 0; i < 2; ++i)
#pragma unroll
        for(int t = 0; t < 2; ++t)
            acc[i][t] = acc_t{0, 0, 0, 0};

    const int nk = (p.K + KT - 1) / KT;
    for(int kt = 0; kt < nk; ++kt)
    {
        const int k0 = kt * KT + lchunk * EPC;
        __attribute__((aligned(16))) elem_t va[EPC];
        __attribute__((aligned(16))) elem_t vb[EPC];
        // ---- A chunk ----
        if constexpr(IM2COL == 0)
        {
            const elem_t* src = A + gm * lay.a_sm + (long)k0 * lay.a_sk;
            if(m_ok && lay.a_sk == 1 && k0 + EPC <= p.K && (reinterpret_cast<uintptr_t>(src) & 15) == 0)
                *reinterpret_cast<i32x4*>(va) = *reinterpret_cast<const i32x4*>(src);
            else
            {
#pragma unroll
                for(int e = 0; e < EPC; ++e)
                    va[e] = (m_ok && k0 + e < p.K) ? src[(long)e * lay.a_sk] : (elem_t)0;
            }
        }
        else
        {
            // k -> ([z,] y, x, c), c fastest; then step element by element
            uint32_t kyx = (uint32_t)k0;
            int z = 0;
            if constexpr(IM2COL == 2)
            {
                z   = (int)magic_div(kyx, p.cv.div_yxc);
                kyx = kyx - (uint32_t)z * p.cv.div_yxc.d;
            }
            int y            = (int)magic_div(kyx, p.cv.div_xc);
            const uint32_t r = kyx - (uint32_t)y * p.cv.div_xc.d;
            int x            = (int)magic_div(r, p.cv.div_c);
            int c            = (int)(r - (uint32_t)x * p.cv.div_c.d);
#pragma unroll
            for(int e = 0; e < EPC; ++e)
            {
                const int hi = hi0 + y * p.cv.dH, wi = wi0 + x * p.cv.dW;
                bool ok = m_ok && k0 + e < p.K && (uint32_t)hi < (uint32_t)p.cv.Hi && (uint32_t)wi < (uint32_t)p.cv.Wi;
                long pix = img;
                if constexpr(IM2COL == 2)
                {
                    const int d = d0 + z * p.cv.dD;
                    ok          = ok && (uint32_t)d < (uint32_t)p.cv.Di;
                    pix         = img * p.cv.Di + d;
                }
                va[e] = ok ? A[((pix * p.cv.Hi + hi) * p.cv.Wi + wi) * p.cv.C + c] : (elem_t)0;
                if(++c == p.cv.C)
                {
                    c = 0;
                    if(++x == lay.X)
                    {
                        x = 0;
                        if(++y == lay.Y)
                            y = 0, ++z;
                    }
                }
            }
        }
        // ---- B chunk ----
        {
            const elem_t* src = B + gn * lay.b_sn + (long)k0 * lay.b_sk;
            if(n_ok && lay.b_sk == 1 && k0 + EPC <= p.K && (reinterpret_cast<uintptr_t>(src) & 15) == 0)
                *reinterpret_cast<i32x4*>(vb) = *reinterpret_cast<const i32x4*>(src);
            else
            {
#pragma unroll
                for(int e = 0; e < EPC; ++e)
                    vb[e] = (n_ok && k0 + e < p.K) ? src[(long)e * lay.b_sk] : (elem_t)0;
            }
        }
        __syncthreads(); // the previous K tile has been read by every wave
        *reinterpret_cast<i32x4*>(sa + lrow * PITCH + lchunk * 16) = *reinterpret_cast<const i32x4*>(va);
        *reinterpret_cast<i32x4*>(sb + lrow * PITCH + lchunk * 16) = *reinterpret_cast<const i32x4*>(vb);
        __syncthreads();
        i32x4 af[2], bf[2];
#pragma unroll
        for(int i = 0; i < 2; ++i)
        {
            af[i] = *reinterpret_cast<const i32x4*>(sa + (wm * 32 + 16 * i + (lane & 15)) * PITCH + (lane >> 4) * 16);
            bf[i] = *reinterpret_cast<const i32x4*>(sb + (wn * 32 + 16 * i + (lane & 15)) * PITCH + (lane >> 4) * 16);
        }
#pragma unroll
        for(int i = 0; i < 2; ++i)
#pragma unroll
            for(int t = 0; t < 2; ++t)
            {
                if constexpr(DT == DT_I8)
                    acc[i][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bf[t], af[i], acc[i][t], 0, 0, 0);
                else if constexpr(DT == DT_BF16)
                    acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, bf[t]),
                                                                     __builtin_bit_cast(bf16x8, af[i]), acc[i][t], 0, 0, 0);
                else
                    acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, bf[t]),
                                                                    __builtin_bit_cast(f16x8, af[i]), acc[i][t], 0, 0, 0);
            }
    }

    // ---- epilogue, element by element: lane owns row (lane % 16), columns 4 * (lane / 16) .. + 3 of every MFMA tile
    const _Float16* d0p = reinterpret_cast<const _Float16*>(p.d0);
    const _Float16* d1p = reinterpret_cast<const _Float16*>(p.d1);
#pragma unroll
    for(int i = 0; i < 2; ++i)
    {
        const long m = (long)tm * 64 + wm * 32 + 16 * i + (lane & 15);
#pragma unroll
        for(int t = 0; t < 2; ++t)
#pragma unroll
            for(int j = 0; j < 4; ++j)
            {
                const long n = (long)tn * 64 + wn * 32 + 16 * t + 4 * (lane >> 4) + j;
                if(m >= p.M || n >= p.N)
                    continue;
                const long ci = g * p.bsc + m * p.ldc + n;
                if constexpr(DT == DT_I8)
                {
                    const int v = acc[i][t][j];
                    const int o = epi_per_column_scale(p.epi)
                                      ? mul2_clamp(v, reinterpret_cast<const float*>(p.d0)[n], p.epi == EPI_RELU_MUL2_CLAMP)
                                  : p.epi == EPI_REQUANT_RND ? requant_rnd(v, p.scale_gemm, p.scale_relu)
                                  : p.epi == EPI_REQUANT_CK  ? requant_ck(v, p.scale_gemm, p.scale_relu)
                                                             : v;
                    reinterpret_cast<int8_t*>(p.c)[ci] = (int8_t)o;
                }
                else if constexpr(DT == DT_BF16)
                    reinterpret_cast<__bf16*>(p.c)[ci] = (__bf16)acc[i][t][j];
                else
                {
                    float v = acc[i][t][j];
                    if(p.epi != EPI_PASSTHROUGH)
                        v = epi_f16_value(p.epi, v, (float)d0p[m * p.ldd0 + n],
                                          epi_has_d1(p.epi) ? (float)d1p[m * p.ldd1 + n] : 0.0f, p.scale_gemm,
                                          p.scale_relu);
                    reinterpret_cast<_Float16*>(p.c)[ci] = (_Float16)v;
                }
            }
    }
}

// dt: DT_*, im2col: 0 (dense A), 1 (one or two spatial dimensions), 2 (three). The grid is
// (C tiles of 64 x 64, batches); GemmArgs::tiles_m / tiles_n must be set for 64 x 64 tiles.
hipError_t launch_generic(int dt, int im2col, const GemmArgs& a, const GenericLayout& lay, hipStream_t s);

} // namespace ckx
