// C ABI of the library (declared in include/ckx.h): argument validation, instance
// selection and kernel launch. No allocation, no synchronisation, no CPU fallback: a
// request no kernel instance covers is reported as CKX_UNSUPPORTED.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <string>

#include "ckx.h"
#include "gemm_tile.hpp"
#include "tile_launch.hpp"
#include "conv_rows.hpp"
#include "gemm_gemm.hpp"
#include "conv_patch.hpp"
#include "conv_patch_wide.hpp"
#include "conv_pointwise.hpp"
#include "conv_stem.hpp"
#include "gemm_skinny.hpp"
#include "gemm_generic.hpp"

// Workspace of ckx_gemm_i8_splitk_noalloc: device memory that belongs to the library, one copy per GPU,
// held from the time the code object is loaded on that GPU until the process ends. In host code the name
// below is only a handle for hipGetSymbolAddress -- it is not a device address; kernels get the pointer
// that static_workspace() returns.
static __device__ __align__(256) unsigned char scratch[CKX_STATIC_WORKSPACE_BYTES];

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& msg)
{
    g_last_error = msg;
    return code;
}

int hip_fail(hipError_t e, const char* what)
{
    return fail(CKX_HIP_ERROR, std::string(what) + ": " + hipGetErrorString(e));
}

// Device address of `scratch` on the current GPU, looked up once per device (every GPU has its own copy of
// the array at its own address). No allocation: hipGetSymbolAddress only resolves the loaded symbol.
int static_workspace(void** out)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* ptrs[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if(e != hipSuccess)
        return hip_fail(e, "hipGetDevice");
    if(dev < 0 || dev >= kMaxDevices)
        return fail(CKX_UNSUPPORTED, "device ordinal beyond the static workspace table");
    std::lock_guard<std::mutex> lock(mu);
    if(!ptrs[dev])
    {
        void* p = nullptr;
        e       = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if(e != hipSuccess || !p)
            return hip_fail(e, "hipGetSymbolAddress(static workspace)");
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return CKX_OK;
}

// int8 outputs at least this large are stored non-temporally (measured on the N256 C256->K512
// 1x1 s2 conv: int8, 103 MB of output, 68.4 us -> 65.0 us; fp16 outputs get SLOWER, 105 -> 127 us,
// so they always use plain stores)
long stream_output_bytes()
{
    // CKX_STREAM_OUTPUT_BYTES overrides the threshold (tuning knob; 0 = always, -1 = never)
    static long v = [] {
        const char* e = std::getenv("CKX_STREAM_OUTPUT_BYTES");
        long t        = e ? std::atol(e) : (64l << 20);
        return t < 0 ? (1l << 62) : t;
    }();
    return v;
}

ckx::MagicDiv make_magic(uint32_t d)
{
    // include/ck/utility/magic_division.hpp:28-54
    uint32_t shift = 0;
    while(shift < 32 && (1ull << shift) < d)
        ++shift;
    const uint64_t one = 1;
    ckx::MagicDiv m;
    m.mul   = (uint32_t)(((one << 32) * ((one << shift) - d)) / d + 1);
    m.shift = shift;
    m.d     = d;
    return m;
}

// ------------------------------------------------------------ tile instances
using ckx::launch_tile;
using ckx::num_cus;
using ckx::tile_launch_fn;

template <int DT>
hipError_t launch_reduce(const ckx::GemmArgs& a, hipStream_t s)
{
    const long groups = (long)a.M * ((a.N + 15) / 16);
    hipLaunchKernelGGL((ckx::splitk_reduce_kernel<DT>), dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s, a);
    return hipGetLastError();
}

struct TileInstance
{
    const char* name;
    int bm, bn, threads, lds;
    float eff; // measured MFMA throughput of this tile shape relative to the 256x256 one
    tile_launch_fn dense_i8, dense_f16, conv_i8, conv_f16, dense_bf16;
    tile_launch_fn dense_f16_fused, conv_f16_fused; // fp16 with the add / ReLU epilogues and D operands
    tile_launch_fn dense_i8_fused, conv_i8_fused;   // int8 with the per-column requant scales as D operand
};

#define CKX_TILE(BM, BN, WM, WN, NST, EFF)                                                         \
    TileInstance{                                                                                  \
        "MI355X_Mfma16_Tile<" #BM ", " #BN ", 128B x" #NST ", waves " #WM "x" #WN ">", BM, BN,           \
            WM* WN * 64, NST*(BM + BN) * 128, EFF, &launch_tile<ckx::DT_I8, BM, BN, WM, WN, 128, NST, false>, \
            &launch_tile<ckx::DT_F16, BM, BN, WM, WN, 128, NST, false>,                               \
            &launch_tile<ckx::DT_I8, BM, BN, WM, WN, 128, NST, true>,                                 \
            &launch_tile<ckx::DT_F16, BM, BN, WM, WN, 128, NST, true>,                                \
            &launch_tile<ckx::DT_BF16, BM, BN, WM, WN, 128, NST, false>,                              \
            &launch_tile<ckx::DT_F16, BM, BN, WM, WN, 128, NST, false, false, false, true>,           \
            &launch_tile<ckx::DT_F16, BM, BN, WM, WN, 128, NST, true, false, false, true>,            \
            &launch_tile<ckx::DT_I8, BM, BN, WM, WN, 128, NST, false, false, false, true>,            \
            &launch_tile<ckx::DT_I8, BM, BN, WM, WN, 128, NST, true, false, false, true>              \
    },

const TileInstance kTiles[] = {CKX_FOR_EACH_TILE(CKX_TILE)};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

// Launch plan: which tile instance, and into how many K runs each C tile is cut (split-K).
struct Plan
{
    int tile   = 0;
    int ksplit = 1;
    int nk_per = 0;
};

// Which body runs the 256 x 256 tile instance on a dense K-contiguous GEMM with a plain epilogue: 0 chooses (below), 4 / 8
// force the four-wave / eight-wave kernel wherever the four-wave one applies (tuning / test knob; CKX_BIG_TILE_WAVES in
// the environment is read on the first call only).
std::atomic<int> g_big_tile_waves{-1};
int big_tile_waves()
{
    int v = g_big_tile_waves.load(std::memory_order_relaxed);
    if(v < 0)
    {
        const char* e = std::getenv("CKX_BIG_TILE_WAVES");
        v             = e ? std::atoi(e) : 0;
        v             = (v == 4 || v == 8) ? v : 0;
        g_big_tile_waves.store(v, std::memory_order_relaxed);
    }
    return v;
}
// The four-wave body (one wave per SIMD, 128 x 128 wave tiles) has the faster K loop -- 18.0 against 18.9 cycles per
// MFMA -- and, for 16-bit outputs, the faster stores (64-byte runs): measured ahead or level at every K for fp16 / bf16.
// Its int8 epilogues have nothing to overlap their table reads with (one wave per SIMD) and it does not prefetch across
// tiles: over the audited int8 problems it is 5 - 18 % behind at 8 K tiles, 2 % at 16, 3 - 6 % ahead from 32 on with one
// tile per CU; with several tiles per CU level at 32 (4096 x 11008 x 4096: 1 % behind), level at 48, 1 - 3 % ahead at 64.
bool four_wave_body_pays(int dt, int K, long tiles)
{
    const int waves = big_tile_waves();
    if(waves)
        return waves == 4;
    // (a single K tile: the four-wave body's plain epilogues run inside a last K tile of their own, all zeros here)
    if((long)K * (dt == ckx::DT_I8 ? 1 : 2) <= 128)
        return false;
    // (fp16 / bf16: it does not prefetch across tiles either, which shows on short K loops with several tiles per CU --
    // 200704 x 256 x 512, eight K tiles, three tiles per CU: 87.3 against 82.6 us; with 1.5 tiles per CU it is ahead:
    // 12544 x 2048 x 512 33.7 against 35.2, and from sixteen K tiles on everywhere measured)
    if(dt != ckx::DT_I8)
        return !(((long)K * 2 + 127) / 128 <= 8 && tiles >= 3l * num_cus());
    return ((long)K + 127) / 128 >= (tiles > num_cus() ? 48 : 32);
}

// CKX_KSPLIT=n forces n K runs where the problem allows it (tuning / test knob). The environment is read on the first
// call only; ckx_set_forced_k_runs() changes the value afterwards (tests force several splits in one process).
std::atomic<int> g_force_ksplit{-1};
int force_ksplit()
{
    int v = g_force_ksplit.load(std::memory_order_relaxed);
    if(v < 0)
    {
        const char* e = std::getenv("CKX_KSPLIT");
        v             = e ? std::atoi(e) : 0;
        v             = v < 0 ? 0 : v;
        g_force_ksplit.store(v, std::memory_order_relaxed);
    }
    return v;
}

// Choice by a small cost model (microseconds on a 256-CU part): work units (C tile x K run) are
// processed in rounds of 256 * (workgroups that fit a CU's 160 KB LDS and 2048 threads); a round
// costs the unit's share of MFMA time, scaled by how well that tile shape feeds the MFMA pipe,
// plus a fixed prologue/epilogue term that co-resident workgroups overlap. Split-K adds the
// second pass (launch + slice traffic) and is only considered when a workspace is available.
// K runs actually used for a requested KBatch: every run must get at least one 128-byte K tile
int splitk_runs(int kbytes, int k_batch)
{
    const int nk = (kbytes + 127) / 128 > 0 ? (kbytes + 127) / 128 : 1;
    k_batch      = k_batch > 8 ? 8 : k_batch;
    for(int sp = k_batch; sp > 1; --sp)
        if((long)((nk + sp - 1) / sp) * (sp - 1) < nk)
            return sp;
    return 1;
}

// k_batch > 0: the caller fixed the number of K runs (DeviceGemmSplitK's KBatch)
// kmajor: a K-major operand (A column-major / B row-major) -- only the tiles of 64 rows and more
// conv: A is gathered (im2col); taps > 1: with several filter taps the 8-wave 256 x 64 tile measures ahead of the
// 128 x 64 one by 10 - 17 % (ResNet-like layers at N = 32 and 256), which the GEMM-calibrated figures did not say; the
// 1 x 1 layers of the same networks follow the GEMM figures (256 x 64 rated up sent C 256 -> K 128 at 56 x 56 to it, 20 %
// behind the 256 x 128 tile)
// d_epilogue: a conv launch with D operands (bias / residual). On K loops of a few tiles the 128 x 128 instance -- two
// co-resident workgroups of one wave per SIMD, each held at the epilogue's wait for its D values with nobody to cover
// for it -- measured 30 - 100 % behind its plain self (C 256 -> K 128, 1x1, 56 x 56, N = 256: 169 us against 128; the
// 256 x 128 instance 132 against 127), so it is left out there.
Plan make_plan(long M, int N, int kbytes, int only_tile, long workspace_bytes, int k_batch = 0, bool kmajor = false,
               bool conv = false, int taps = 2, bool d_epilogue = false)
{
    Plan best;
    double best_us  = 1e30;
    const long cus  = num_cus(); // (the time constants below were measured on a 256-CU part)
    const int nk    = (kbytes + 127) / 128 > 0 ? (kbytes + 127) / 128 : 1;
    const int force = k_batch > 0 ? splitk_runs(kbytes, k_batch) : force_ksplit();
    for(int i = 0; i < kNumTiles; ++i)
    {
        if(only_tile >= 0 && i != only_tile)
            continue;
        const TileInstance& t = kTiles[i];
        if(kmajor && t.bm < 64)
            continue;
        if(conv && d_epilogue && only_tile < 0 && t.bm == 128 && t.bn == 128 && nk <= 8)
            continue;
        const long tiles      = (long)((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn);
        for(int sp = 1; sp <= 8; ++sp)
        {
            const int nk_per = (nk + sp - 1) / sp;
            if(sp > 1 && ((long)nk_per * (sp - 1) >= nk || (long)sp * M * N * 4 > workspace_bytes))
                continue;
            if(force > 0 && sp != force && !(sp == 1 && ((long)((nk + force - 1) / force) * (force - 1) >= nk ||
                                                          (long)force * M * N * 4 > workspace_bytes)))
                continue;
            const long units = tiles * sp;
            int per_cu       = 160 * 1024 / t.lds;
            per_cu           = per_cu > 2048 / t.threads ? 2048 / t.threads : per_cu;
            per_cu           = per_cu > 4 ? 4 : per_cu;
            per_cu           = per_cu * cus > units ? (int)((units + cus - 1) / cus) : per_cu;
            const long rounds = (units + cus * per_cu - 1) / (cus * per_cu);
            // one K-tile iteration costs its MFMA time, but never less than the barrier + load
            // latency of the two-stage pipeline (~0.42 us measured on small tiles)
            const double eff = conv && taps > 1 && t.bm == 256 && t.bn == 64 ? t.eff * 1.1 : t.eff;
            double iter_us   = per_cu * (t.bm * t.bn / 65536.0) / eff * 1.1;
            const int nst  = t.lds / ((t.bm + t.bn) * 128);
            const double floor_us = nst > 2 ? 0.30 : 0.42; // (four stages: 0.33 measured over 32 K tiles, 0.26 over 64)
            iter_us        = iter_us < floor_us ? floor_us : iter_us;
            // three and more co-resident workgroups pull their K tiles through ONE CU's load path: 105 GB/s out of L2
            // with every CU busy (measured with a streaming probe), 85 in a kernel that also computes. Without this term
            // 128 x 64 tiles at three per CU were rated 43 us on fp16 512 x 11008 x 4096 and took 60 (256 x 128: 48).
            // (GEMM launches only: an im2col A operand re-reads its pixels out of L1 / L2 tap after tap, and with the term
            // the 3-D layer 4 x 28^3 x 64 -> 256, stride 2, went from the 64 x 64 tile, 24.7 us, to 256 x 64 at 35.9)
            if(per_cu >= 3 && !conv)
            {
                const double load_us = per_cu * (double)(t.bm + t.bn) * 128.0 / 85.0e3;
                iter_us              = iter_us < load_us ? load_us : iter_us;
            }
            double us      = rounds * (iter_us * nk_per + 6.0 / per_cu + 2.0);
            // a single, partly filled round of one four-stage workgroup per CU: measured fixed cost ~4 us, not 8 (M = 64,
            // N = 11008, K = 4096 int8 on the four-stage 64 x 64 tile: 14.4 us = 3.8 + 0.33 per K tile; the 8 sent
            // such problems to one-wave tiles at 20 us)
            if(rounds == 1 && per_cu == 1 && sp == 1 && (nst > 2 || (conv && t.threads == 512)))
                us -= 4.0;
            if(sp > 1)
            {
                // second launch + slice write/read (measured ~2 TB/s effective), and a split has to
                // promise a clear win: the single-pass estimate is the better calibrated one
                us += 3.0 + (sp + 0.25) * M * (double)N * 4 / 2.0e6;
                if(force <= 0)
                    us *= 1.5;
            }
            if(us < best_us)
                best_us = us, best.tile = i, best.ksplit = sp, best.nk_per = nk_per;
        }
    }
    if(best.nk_per == 0)
        best.nk_per = nk;
    // Cache-resident problems of one round of 64 x 64 tiles (M = N = K = 1024 int8: 256 tiles, 3 MB): measured
    // 5.9 us on the two-stage 64 x 64 instance against 7.3 us on the four co-resident one-wave workgroups per CU the
    // estimate above prefers (every one of those loads its own copy of the B rows), 7.7 / 10.6 us on larger tiles.
    if(only_tile < 0 && !kmajor && k_batch == 0 && best.ksplit == 1 && nk <= 16 &&
       ((long)M + N) * kbytes + (long)M * N <= (8l << 20))
    {
        const long t64 = (long)((M + 63) / 64) * ((N + 63) / 64);
        // (and the two-stage instance also where the estimate picks its four-stage twin: 64 x 2048 x 2048 7.9 against
        // 8.6 us -- the deeper pipeline pays when the operands stream from HBM, not out of L2)
        const bool twin = kTiles[best.tile].bm == 64 && kTiles[best.tile].bn == 64 && kTiles[best.tile].lds > 2 * 128 * 128;
        for(int i = 0; i < kNumTiles; ++i)
            if(kTiles[i].bm == 64 && kTiles[i].bn == 64 && kTiles[i].lds == 2 * 128 * 128 &&
               (twin || (t64 > 128 && t64 <= 256 && kTiles[best.tile].bm * kTiles[best.tile].bn < 64 * 64)))
                best.tile = i;
    }
    return best;
}

// ---------------------------------------------------------- skinny instances
struct SkinnyInstance
{
    const char* name;
    int max_m, cols;
    tile_launch_fn i8, f16, bf16;
};

template <int DT, int MT, int NW, int KU, int NT>
hipError_t launch_skinny(const ckx::GemmArgs& a, int grid, hipStream_t s)
{
    hipLaunchKernelGGL((ckx::gemm_skinny_kernel<DT, MT, NW, KU, NT>), dim3(grid), dim3(NW * 64), 0, s, a);
    return hipGetLastError();
}

#define CKX_SKINNY(MT, NW, KU, NT)                                                                          \
    {                                                                                                       \
        "MI355X_Mfma16_Skinny<rows " #MT "x16, cols " #NT "x16, waves " #NW ", unroll " #KU ">", MT * 16, NT * 16, \
            &launch_skinny<ckx::DT_I8, MT, NW, KU, NT>, &launch_skinny<ckx::DT_F16, MT, NW, KU, NT>,             \
            &launch_skinny<ckx::DT_BF16, MT, NW, KU, NT>                                                    \
    }

// the weight-streaming instance for up to 128 rows (gemm_astream.hpp): A tiles of all rows in LDS, requested by loader
// waves; B straight into the compute waves' registers; the whole K extent per workgroup
#define CKX_ASTREAM(NT)                                                                                                \
    {                                                                                                                  \
        "MI355X_Mfma16_Stream<rows 8x16, cols " #NT "x16, 4 compute + 4 loader waves, A tiles in LDS, B in registers>", 128, NT * 16, \
            ckx::astream_launcher(ckx::DT_I8, NT), ckx::astream_launcher(ckx::DT_F16, NT),                              \
            ckx::astream_launcher(ckx::DT_BF16, NT)                                                                    \
    }

const SkinnyInstance kSkinny[] = {
    CKX_SKINNY(1, 8, 4, 1),
    CKX_SKINNY(2, 8, 4, 1),
    CKX_SKINNY(4, 8, 2, 1),
    CKX_SKINNY(1, 16, 2, 1),
    CKX_SKINNY(1, 8, 2, 4),
    CKX_SKINNY(1, 8, 2, 2),
    CKX_SKINNY(2, 8, 2, 4),
    CKX_SKINNY(2, 8, 2, 2),
    CKX_ASTREAM(3),
};
constexpr int kAStream = 8; // (position in kSkinny)
constexpr int kNumSkinny    = sizeof(kSkinny) / sizeof(kSkinny[0]);
// the element-granular instance (gemm_generic.hpp) closes every GEMM and conv instance list: any extent, leading
// dimension, channel count and base address, all four GEMM layouts, every epilogue of the data type
constexpr int kGenericGemmInstance = kNumTiles + kNumSkinny;
constexpr int kNumGemmInsts        = kNumTiles + kNumSkinny + 1;
const char* const kGenericName     = "MI355X_Mfma16_Generic<64, 64, one k-step, waves 2x2, element-wise loads>";

const char* family_prefix(int op)
{
    switch(op)
    {
    case CKX_OP_GEMM_I8: return "DeviceGemm_i8_i8_i8_mk_nk_mn";
    case CKX_OP_GEMM_F16: return "DeviceGemm_f16_f16_f16_mk_nk_mn";
    case CKX_OP_CONV2D_FWD_I8: return "DeviceConv2dFwd_i8_nhwc_kyxc_nhwk";
    case CKX_OP_CONV2D_FWD_F16: return "DeviceConv2dFwd_f16_nhwc_kyxc_nhwk";
    case CKX_OP_BATCHED_GEMM_GEMM: return "DeviceBatchedGemmGemm_f16_gmk_gnk_gno_gmo";
    case CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM: return "DeviceBatchedGemmSoftmaxGemm_f16_gmk_gnk_gno_gmo";
    case CKX_OP_GEMM_SPLITK: return "DeviceGemmSplitK_mk_nk_mn";
    case CKX_OP_GEMM_BF16: return "DeviceGemm_bf16_bf16_bf16_mk_nk_mn";
    default: return nullptr;
    }
}

// Operands of the fused add epilogues (fp16): D0 / D1 are [M,N] row-major, row strides in elements
struct DOperands
{
    const void* d0 = nullptr;
    const void* d1 = nullptr;
    int ldd0 = 0, ldd1 = 0;
};

// the fp16 add / ReLU functors with fp16 D operands; the int8 functors with a per-column fp32 scale row as D0
bool f16_fused(int epi)
{
    return (epi >= CKX_EPI_ADD_RELU && epi <= CKX_EPI_CSHUFFLE_ADD_RELU) || epi == CKX_EPI_BILINEAR ||
           epi == CKX_EPI_ADD_ADD_FASTGELU;
}
bool uses_d1(int epi) { return epi == CKX_EPI_ADD_RELU_ADD || epi == CKX_EPI_ADD_ADD_FASTGELU; }
// the CDE operations of ckx_gemm_f16_multiple_d (the bilinear one has its scalars and its own entry point)
bool f16_cde_op(int epi) { return f16_fused(epi) && epi != CKX_EPI_BILINEAR; }
bool per_column_scale(int epi) { return epi == CKX_EPI_MUL2_CLAMP || epi == CKX_EPI_RELU_MUL2_CLAMP; }

bool epilogue_fits_dtype(int es, int epi)
{
    if(es == 1)
        return (epi >= CKX_EPI_PASSTHROUGH && epi <= CKX_EPI_REQUANT_RND) || per_column_scale(epi);
    return epi == CKX_EPI_PASSTHROUGH || f16_fused(epi);
}

int check_d_operands(int epi, int N, const DOperands& d)
{
    if(epi < CKX_EPI_ADD_RELU)
        return CKX_OK;
    if(per_column_scale(epi))
    {
        if(!d.d0)
            return fail(CKX_INVALID_VALUE, "null D operand pointer");
        if(d.ldd0 != 0)
            return fail(CKX_UNSUPPORTED, "the requant scales are one row of N floats: D0 stride 0 (broadcast over the rows)");
        if(reinterpret_cast<uintptr_t>(d.d0) & 3)
            return fail(CKX_UNSUPPORTED, "operands must be aligned to their element size");
        return CKX_OK;
    }
    if(!d.d0 || (uses_d1(epi) && !d.d1))
        return fail(CKX_INVALID_VALUE, "null D operand pointer");
    if((d.ldd0 != 0 && d.ldd0 < N) || (uses_d1(epi) && d.ldd1 != 0 && d.ldd1 < N) || d.ldd0 < 0 ||
       d.ldd1 < 0)
        return fail(CKX_UNSUPPORTED, "D stride must be 0 (broadcast row) or at least N");
    return CKX_OK;
}

// Problems outside the vectorised instances' reach: a contiguous extent or a leading dimension of A or B that is not
// a whole 16-byte vector (the reference's KPadding / MNKPadding territory), D-operand epilogues on K-major operands
bool gemm_needs_generic(int dt, int M, int N, int K, int sa, int sb, bool ta, bool tb, int epi)
{
    const int es = dt == ckx::DT_I8 ? 1 : 2;
    return ((long)(ta ? M : K) * es) % 16 || ((long)(tb ? N : K) * es) % 16 || ((long)sa * es) % 16 ||
           ((long)sb * es) % 16 || ((ta || tb) && (f16_fused(epi) || per_column_scale(epi)));
}

int check_gemm_shape(int dt, int M, int N, int K, int sa, int sb, int sc, int al, int bl, int cl, int epi,
                     int instance)
{
    const int es = dt == ckx::DT_I8 ? 1 : 2;
    if(M < 0 || N < 0 || K < 0)
        return fail(CKX_INVALID_VALUE, "negative GEMM dimension");
    if(instance != CKX_INSTANCE_AUTO && (instance < 0 || instance >= kNumGemmInsts))
        return fail(CKX_INVALID_VALUE, "no such instance");
    if(instance >= kNumTiles && instance < kGenericGemmInstance && M > kSkinny[instance - kNumTiles].max_m)
        return fail(CKX_UNSUPPORTED, "this skinny instance covers fewer rows than M");
    if(epi < CKX_EPI_PASSTHROUGH || epi > CKX_EPI_ADD_ADD_FASTGELU)
        return fail(CKX_INVALID_VALUE, "unknown epilogue");
    if(!epilogue_fits_dtype(es, epi) || (dt == ckx::DT_BF16 && epi != CKX_EPI_PASSTHROUGH))
        return fail(CKX_UNSUPPORTED, "epilogue not available for this dtype");
    if((al != CKX_ROW_MAJOR && al != CKX_COL_MAJOR) || (bl != CKX_ROW_MAJOR && bl != CKX_COL_MAJOR))
        return fail(CKX_INVALID_VALUE, "unknown layout");
    if(cl != CKX_ROW_MAJOR)
        return fail(CKX_UNSUPPORTED, "C is row-major in every instance (as in the reference's instance lists)");
    // K-major operands: A column-major (element (m,k) at k*sa + m), B row-major ((k,n) at k*sb + n)
    const bool ta = al == CKX_COL_MAJOR, tb = bl == CKX_ROW_MAJOR;
    // what only the element-granular instance takes (AUTO sends it there)
    const bool fast = instance != CKX_INSTANCE_AUTO && instance != kGenericGemmInstance;
    if(fast && (ta || tb) && (f16_fused(epi) || per_column_scale(epi)))
        return fail(CKX_UNSUPPORTED, "the D-operand epilogues of this instance are built for A row-major, B column-major");
    if(fast && (ta || tb) && !ckx::layout_tile(dt, instance, ta, tb))
        return fail(CKX_UNSUPPORTED, "this instance has no variant for a K-major operand (tiles of 64 rows and more do)");
    if(sa < (ta ? M : K) || sb < (tb ? N : K) || sc < N)
        return fail(CKX_UNSUPPORTED, "stride smaller than the contiguous extent");
    if(fast && gemm_needs_generic(dt, M, N, K, sa, sb, ta, tb, epi))
        return fail(CKX_UNSUPPORTED, "the contiguous extents of A and B and their strides must be multiples of 16 bytes "
                                     "for this instance (the element-wise instance and AUTO take any)");
    if((long)(ta ? K : M) * sa * es >= (1l << 31) || (long)(tb ? K : N) * sb * es >= (1l << 31) ||
       (long)M * sc * es >= (1l << 31))
        return fail(CKX_UNSUPPORTED, "operands of 2 GiB or more are not addressed");
    return CKX_OK;
}

// workspace need of the launch plan for this GEMM (0: none)
long gemm_workspace_bytes(int dt, int M, int N, int K, int instance)
{
    const int es = dt == ckx::DT_I8 ? 1 : 2;
    // (up to 16 rows go to the skinny kernels, which take none -- except few columns under a long K: see run_gemm)
    const bool few_cols = M >= 8 && (N + 15) / 16 < (M > 16 ? 257 : 128) && (long)K * es >= 16384;
    if(M <= 0 || N <= 0 || (instance == CKX_INSTANCE_AUTO && M <= 16 && !few_cols) || instance >= kNumTiles ||
       ((long)K * es) % 16)
        return 0;
    const Plan pl = make_plan(M, N, K * es, instance, 1l << 60);
    return pl.ksplit > 1 ? (long)pl.ksplit * M * N * 4 : 0;
}

// strided-batch part of the argument check (DeviceBatchedGemm)
// bytes from the first to one past the last element of an operand of `rows` rows of `cols` contiguous elements
long operand_extent(int batch, long bs, int rows, int cols, int stride, int es)
{
    return rows > 0 && cols > 0 ? ((long)(batch - 1) * bs + (long)(rows - 1) * stride + cols) * es : 0;
}

int check_batch(int dt, int M, int N, int K, int sa, int sb, int sc, bool ta, bool tb, int epi, int instance,
                int k_batch, int batch, long bsa, long bsb, long bsc)
{
    if(batch < 0)
        return fail(CKX_INVALID_VALUE, "negative batch count");
    if(batch > 1)
    {
        const int es = dt == ckx::DT_I8 ? 1 : 2;
        if(instance >= kNumTiles && instance != kGenericGemmInstance)
            return fail(CKX_UNSUPPORTED, "batched GEMM runs on the tile instances and the element-wise instance");
        if(epi >= CKX_EPI_ADD_RELU || k_batch > 1)
            return fail(CKX_UNSUPPORTED, "batched GEMM has neither D operands nor a K split");
        if(bsa < 0 || bsb < 0 || bsc < 0)
            return fail(CKX_UNSUPPORTED, "batch strides must be non-negative");
        if(instance != CKX_INSTANCE_AUTO && instance != kGenericGemmInstance && ((bsa * es) % 16 || (bsb * es) % 16))
            return fail(CKX_UNSUPPORTED, "batch strides of A and B must be multiples of 16 bytes for this instance");
        if(batch > 65535 && (instance == kGenericGemmInstance || (bsa * es) % 16 || (bsb * es) % 16 ||
                             gemm_needs_generic(dt, M, N, K, sa, sb, ta, tb, epi)))
            return fail(CKX_UNSUPPORTED, "the element-wise instance takes at most 65535 batches");
        if(bsc < (long)(M - 1) * sc + N && M > 0 && N > 0)
            return fail(CKX_UNSUPPORTED, "C batches overlap");
        const long ea = operand_extent(batch, bsa, ta ? K : M, ta ? M : K, sa, es);
        const long eb = operand_extent(batch, bsb, tb ? K : N, tb ? N : K, sb, es);
        if(ea >= (1l << 31) || eb >= (1l << 31) || ((long)(batch - 1) * bsc + (long)M * sc) * es >= (1l << 31))
            return fail(CKX_UNSUPPORTED, "operands of 2 GiB or more are not addressed");
    }
    return CKX_OK;
}

// The instance (index into the GEMM family list) and K runs a launch of a vector-aligned problem uses: the automatic
// choice for instance == CKX_INSTANCE_AUTO, else the given instance with its own K split. Pure host logic, shared by the
// launcher and ckx_gemm_plan(). workspace_bytes: usable workspace (0: none, or unaligned).
struct GemmChoice
{
    int instance;
    int ksplit;
    int nk_per;
};

GemmChoice choose_gemm(int dt, int M, int N, int K, bool kmajor, int instance, long workspace_bytes, int k_batch, int batch)
{
    const int es = dt == ckx::DT_I8 ? 1 : 2;
    const int nk = ((long)K * es + 127) / 128 > 0 ? (int)(((long)K * es + 127) / 128) : 1;
    if(instance >= kNumTiles)
        return GemmChoice{instance, 1, nk};
    const bool ws = workspace_bytes > 0;
    // 17..64 rows: the tile kernel wins when its C tiles fill the machine, or C tiles x K runs over a long K
    // (17..32 rows since the re-measured audit: fp16 32 x 11008 x 4096 18.3 us on the four-stage 64 x 64 tile against
    // 25.4 on the widest skinny instance, int8 13.8 against 14.3)
    // (64 x 4096 x 11008: 20 against 27 us; at K = 4096 the 64-row skinny instance is ahead, 11.8 against 13.0 us)
    // (fp16, 8..16 rows, many columns and a long K: HBM streaming either way, and the skinny kernels' A re-reads out of
    // L2 show -- 16 x 11008 x 4096 fp16: 21.6 us against 18.2 on the four-stage tile; int8 stays: 12.2 against 13.8)
    // 65 .. 128 rows against a weight matrix of 32 MB and more whose 48-column blocks fill most of the CUs in one round: the
    // weight-streaming instance (A tiles of all rows through LDS by loader waves, B straight into registers, all of K per
    // workgroup, one launch). 128 x 11008 x 4096 int8: 20.1 us against 23.3 with the weights coming out of HBM (eight
    // copies used in turn), 17.2 against 16.5 us when they sit in the Infinity Cache -- weights of a model that does not
    // fit that cache are the case that counts. (A longer K means more of A per byte of B through every CU: at K = 8192 the
    // tile kernel with K runs is ahead, 25.0 against 32.9 us; fp16 doubles the bytes of K as well.)
    const long stream_blocks = (N + 47) / 48;
    if(instance == CKX_INSTANCE_AUTO && !kmajor && batch == 1 && k_batch == 0 && es == 1 && M > 64 && M <= 128 &&
       (long)N * K * es >= (32l << 20) && (long)K * es <= 6144 && stream_blocks >= 160 && stream_blocks <= num_cus())
        return GemmChoice{kNumTiles + kAStream, 1, nk};
    const bool f16_long = es == 2 && M >= 8 && M <= 64 && (long)K * es >= 8192 && (N + 63) / 64 >= 160;
    const bool tile64 = kmajor || f16_long || (M > 16 && M <= 64 &&
                                   ((N + 63) / 64 >= 160 ||
                                    (ws && (long)K * es >= 8192 && make_plan(M, N, K * es, -1, workspace_bytes).ksplit > 1)));
    // few columns and a long K: the skinny kernels have N / 16 workgroups with all of K each, the tile kernel can cut K
    // over the CUs (fp16 32 x 1024 x 8192: 12.4 against 23.3 us, 16 rows 12.1 against 16.2, 8 rows 11.7 against 13.4)
    // (17 rows and more: up to 4096 columns -- fp16 32 x 4096 x 11008 24.6 against 31.9 us)
    const bool few_cols = !kmajor && M >= 8 && M <= 64 && (N + 15) / 16 < (M > 16 ? 257 : 128) && (long)K * es >= 16384 &&
                          ws && make_plan(M, N, K * es, -1, workspace_bytes).ksplit > 1;
    if(instance == CKX_INSTANCE_AUTO && M <= 64 && !tile64 && !few_cols && k_batch == 0 && batch == 1)
    {
        // (the skinny kernels read both operands K-contiguous: other layouts always take the tile kernel)
        // A handful of rows against a big weight matrix is an HBM-streaming problem. Wider
        // workgroups (32 / 64 columns) re-read A from L2 less often, as long as enough workgroups
        // remain to keep every CU pulling on HBM; up to 4 rows A is too small to matter unless the columns are many.
        // (measured: 8 x 11008 x 4096 11.5 against 12.4 us on the 64-column instance, 1 x 11008 x 4096 11.0 against
        // 10.6; 1 and 8 x 16384 x 1024 5.5 against 8.7 / 9.4 us)
        const int n64  = (N + 63) / 64;
        const int wide = M <= 4 ? (n64 >= 256 ? 2 : 0) : n64 >= 160 ? 2 : (M > 8 && (N + 31) / 32 >= 160) ? 1 : 0;
        const int ti   = kNumTiles + (M <= 16 ? (wide == 2 ? 4 : wide == 1 ? 5 : 0) : M <= 32 ? (wide == 2 ? 6 : wide == 1 ? 7 : 1) : 2);
        return GemmChoice{ti, 1, nk};
    }
    // a batch multiplies the C tiles: plan for a problem with that many rows, without a K split
    const Plan pl = batch > 1 ? make_plan((long)M * (batch < 64 ? batch : 64), N, K * es, instance, 0, 1, kmajor)
                              : make_plan(M, N, K * es, instance, workspace_bytes, k_batch, kmajor);
    return GemmChoice{pl.tile, pl.ksplit, pl.nk_per};
}

int run_gemm(int dt, const void* a, const void* b, void* c, int M, int N, int K, int sa, int sb, int sc,
             int al, int bl, int cl, int epi, float sg, float sr, int instance, void* ws, long ws_bytes,
             void* stream, const DOperands& dops = DOperands{}, int k_batch = 0, int batch = 1, long bsa = 0,
             long bsb = 0, long bsc = 0)
{
    int st = check_gemm_shape(dt, M, N, K, sa, sb, sc, al, bl, cl, epi, instance);
    if(st != CKX_OK)
        return st;
    if(k_batch < 0 || k_batch > 8)
        return fail(CKX_UNSUPPORTED, "KBatch must be 1..8");
    if(k_batch > 0 && instance >= kNumTiles && instance != kGenericGemmInstance)
        return fail(CKX_UNSUPPORTED, "the skinny instances split K over their waves, not over runs");
    const bool ta = al == CKX_COL_MAJOR, tb = bl == CKX_ROW_MAJOR, kmajor = ta || tb;
    if((st = check_batch(dt, M, N, K, sa, sb, sc, ta, tb, epi, instance, k_batch, batch, bsa, bsb, bsc)) != CKX_OK)
        return st;
    if(batch == 0)
        return CKX_OK;
    if((st = check_d_operands(epi, N, dops)) != CKX_OK)
        return st;
    if(M == 0 || N == 0)
        return CKX_OK;
    if(!a || !b || !c)
        return fail(CKX_INVALID_VALUE, "null operand pointer");
    const int es = dt == ckx::DT_I8 ? 1 : 2;
    const bool misaligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) != 0 ||
                            (batch > 1 && ((bsa * es) % 16 || (bsb * es) % 16));
    if(instance == kGenericGemmInstance ||
       (instance == CKX_INSTANCE_AUTO && (misaligned || gemm_needs_generic(dt, M, N, K, sa, sb, ta, tb, epi))))
    {
        // element-granular instance: one pass over K whatever KBatch says (the result does not depend on the split)
        if((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c) |
            (f16_fused(epi) ? reinterpret_cast<uintptr_t>(dops.d0) | reinterpret_cast<uintptr_t>(dops.d1) : 0)) & (es - 1))
            return fail(CKX_UNSUPPORTED, "operands must be aligned to their element size");
        ckx::GemmArgs g;
        std::memset(&g, 0, sizeof(g));
        g.a = a, g.b = b, g.c = c;
        g.M = M, g.N = N, g.K = K;
        g.lda = sa, g.ldb = sb, g.ldc = sc;
        g.batch = batch, g.bsa = bsa, g.bsb = bsb, g.bsc = bsc;
        g.epi = epi, g.scale_gemm = sg, g.scale_relu = sr;
        g.d0 = dops.d0, g.d1 = uses_d1(epi) ? dops.d1 : nullptr;
        g.ldd0 = dops.ldd0, g.ldd1 = dops.ldd1;
        g.ksplit  = 1;
        g.tiles_m = (M + 63) / 64, g.tiles_n = (N + 63) / 64;
        if(batch > 65535)
            return fail(CKX_UNSUPPORTED, "the element-granular instance (operands that are not 16-byte aligned vectors) "
                                         "takes at most 65535 batches per launch");
        ckx::GenericLayout lay{};
        lay.a_sm = ta ? 1 : sa, lay.a_sk = ta ? sa : 1;
        lay.b_sn = tb ? 1 : sb, lay.b_sk = tb ? sb : 1;
        hipError_t e = ckx::launch_generic(dt, 0, g, lay, (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kGenericName);
    }
    if(misaligned)
        return fail(CKX_UNSUPPORTED, "A and B (and their batch strides) must be 16-byte aligned for this instance");
    const bool ws_ok    = ws && !(reinterpret_cast<uintptr_t>(ws) & 15);
    const GemmChoice ch = choose_gemm(dt, M, N, K, kmajor, instance, ws_ok ? ws_bytes : 0, k_batch, batch);
    const int ti        = ch.instance;
    if(ti < kNumTiles)
    {
        if(ws && !ws_ok)
            return fail(CKX_INVALID_VALUE, "workspace must be 16-byte aligned");
        if(k_batch > 1 && splitk_runs(K * es, k_batch) > 1 &&
           (!ws || ws_bytes < (long)splitk_runs(K * es, k_batch) * M * N * 4))
            return fail(CKX_INVALID_VALUE, "KBatch > 1 needs a workspace of ckx_gemm_splitk_workspace_bytes()");
    }
    Plan pl;
    pl.tile = ch.instance < kNumTiles ? ch.instance : 0, pl.ksplit = ch.ksplit, pl.nk_per = ch.nk_per;
    ckx::GemmArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = a, g.b = b, g.c = c;
    g.M = M, g.N = N, g.K = K;
    g.lda = sa, g.ldb = sb, g.ldc = sc;
    g.a_bytes    = (uint32_t)operand_extent(batch, bsa, ta ? K : M, ta ? M : K, sa, es);
    g.b_bytes    = (uint32_t)operand_extent(batch, bsb, tb ? K : N, tb ? N : K, sb, es);
    g.batch = batch, g.bsa = bsa, g.bsb = bsb, g.bsc = bsc;
    g.epi        = epi;
    g.scale_gemm = sg;
    g.scale_relu = sr;
    g.nt_store   = es == 1 && (long)M * N * es >= stream_output_bytes();
    g.d0 = dops.d0, g.d1 = uses_d1(epi) ? dops.d1 : nullptr;
    g.ldd0 = dops.ldd0, g.ldd1 = dops.ldd1;
    g.ksplit     = 1;
    if(ti >= kNumTiles)
    {
        const SkinnyInstance& k = kSkinny[ti - kNumTiles];
        hipError_t e = (dt == ckx::DT_I8 ? k.i8 : dt == ckx::DT_BF16 ? k.bf16 : k.f16)(g, (N + k.cols - 1) / k.cols,
                                                                                      (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, k.name);
    }
    const TileInstance& t = kTiles[ti];
    g.tiles_m    = (M + t.bm - 1) / t.bm;
    g.tiles_n    = (N + t.bn - 1) / t.bn;
    g.ksplit     = pl.ksplit;
    g.nk_per     = pl.nk_per;
    g.ws         = ws;
    const bool fused            = f16_fused(epi) && g.ksplit == 1; // (after a K split the second pass applies it)
    // (the functors with a second D tensor stay on the eight-wave body: see the fused epilogue of gemm_w4.hpp)
    // (its buffer resources start 3 KB before the operands and are that much longer: see kImmBias in gemm_w4.hpp)
    const bool w4 = ti == 0 && !kmajor && g.ksplit == 1 && g.a_bytes < (1u << 31) - 4096 && g.b_bytes < (1u << 31) - 4096 &&
                    (epi <= CKX_EPI_REQUANT_RND || (f16_fused(epi) && !uses_d1(epi))) && four_wave_body_pays(dt, K, (long)g.tiles_m * g.tiles_n * (batch > 1 ? batch : 1));
    const tile_launch_fn launch = w4                   ? ckx::w4_tile(dt, fused)
                                  : kmajor             ? ckx::layout_tile(dt, ti, ta, tb)
                                  : dt == ckx::DT_I8   ? (per_column_scale(epi) && g.ksplit == 1 ? t.dense_i8_fused : t.dense_i8)
                                  : dt == ckx::DT_BF16 ? t.dense_bf16
                                  : fused              ? t.dense_f16_fused
                                                       : t.dense_f16;
    if(!launch)
        return fail(CKX_UNSUPPORTED, "no kernel variant for this layout");
    hipError_t e = launch(g, g.tiles_m * g.tiles_n * g.ksplit * batch, (hipStream_t)stream);
    if(e == hipSuccess && g.ksplit > 1)
        e = dt == ckx::DT_I8     ? launch_reduce<ckx::DT_I8>(g, (hipStream_t)stream)
            : dt == ckx::DT_BF16 ? launch_reduce<ckx::DT_BF16>(g, (hipStream_t)stream)
                                 : launch_reduce<ckx::DT_F16>(g, (hipStream_t)stream);
    if(e != hipSuccess)
        return hip_fail(e, t.name);
    return CKX_OK;
}

// ---------------------------------------------------------- input-patch conv kernel
const char* const kPatchName = "MI355X_Mfma16_Patch<3x3, C = K = 64 rows x 56 or C = K = 128 rows x 28, 4 waves, weights in AccVGPRs>";

// the second shape of the instance (conv_patch_wide.hpp): C = K = 128, Wo = 28; plain epilogues and fp16 bias + ReLU
bool conv_patch_wide_applicable(int op, const ckx_conv2d_desc* d, int epi)
{
    const bool epi_ok = op == CKX_OP_CONV2D_FWD_F16 ? (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_ADD_RELU)
                                                    : (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_REQUANT_CK || epi == CKX_EPI_REQUANT_RND);
    return (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && epi_ok && d->C == 128 && d->K == 128 && d->Y == 3 &&
           d->X == 3 && d->stride_h == 1 && d->stride_w == 1 && d->dilation_h == 1 && d->dilation_w == 1 &&
           d->Wo == 28 && d->Ho >= 1 && d->N >= 1 && d->pad_left <= 2 && d->pad_top <= 2;
}

// shapes the input-patch kernels cover (one instantiation per data type and shape: 3x3 taps, Wo = 56 / 28)
bool conv_patch_applicable(int op, const ckx_conv2d_desc* d, int epi)
{
    if(conv_patch_wide_applicable(op, d, epi))
        return true;
    const bool epi_ok = op == CKX_OP_CONV2D_FWD_F16
                            ? (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_ADD_RELU || epi == CKX_EPI_ADD_RELU_ADD)
                            : (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_REQUANT_CK || epi == CKX_EPI_REQUANT_RND ||
                               per_column_scale(epi));
    return (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && epi_ok && d->C == 64 && d->K == 64 && d->Y == 3 &&
           d->X == 3 && d->stride_h == 1 && d->stride_w == 1 && d->dilation_h == 1 && d->dilation_w == 1 &&
           d->Wo == 56 && d->Ho >= 1 && d->N >= 1 && d->pad_left <= 2 && d->pad_top <= 2;
}

// ... and the ones it is chosen for: a workgroup owns whole images, so a small batch leaves CUs idle (N = 32: 54 us
// against 18 us on the 256 x 64 tile instance, whose time grows with N: the curves cross near N = 100)
bool conv_patch_preferred(int op, const ckx_conv2d_desc* d, int epi)
{
    return conv_patch_applicable(op, d, epi) && d->N >= 112;
}

// ---------------------------------------------------------- weight-stationary pointwise conv kernel
const char* const kPointwiseName = "MI355X_Mfma16_Pointwise<1x1, C 256/512 bytes, K 512 per workgroup, 8 waves>";
const char* const kRowsName = "MI355X_Mfma16_Rows<1x1, stride 1, pixels of 64 ... 512 bytes, K <= 256 per workgroup, weights in registers, no LDS>";
constexpr int kConvPatchInstance = kNumTiles, kConvPointwiseInstance = kNumTiles + 1, kConvStemInstance = kNumTiles + 2,
              kConvRowsInstance = kNumTiles + 3, kConvGenericInstance = kNumTiles + 4, kNumConvInsts = kNumTiles + 5;

// ---------------------------------------------------------- stem conv kernel (three input channels)
const char* const kStemName = "MI355X_Mfma16_Stem<7x7, stride 2, pad 3, C 3, K 64, pixels padded to 4 channels in LDS, 4 waves>";
// the first layer of an image network: C = 3, 7 x 7, stride 2, padding 3 on every side, 64 output channels; the LDS holds
// the 13 input rows of a band of four output rows
bool conv_stem_applicable(int op, const ckx_conv2d_desc* d, int epi)
{
    const bool epi_ok = op == CKX_OP_CONV2D_FWD_F16 ? (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_ADD_RELU)
                                                    : (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_REQUANT_CK ||
                                                       epi == CKX_EPI_REQUANT_RND);
    if(!((op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && epi_ok && d->C == 3 && d->K == 64 && d->Y == 7 &&
         d->X == 7 && d->stride_h == 2 && d->stride_w == 2 && d->dilation_h == 1 && d->dilation_w == 1 && d->pad_top == 3 &&
         d->pad_left == 3 && d->pad_bottom == 3 && d->pad_right == 3 && d->N >= 1 && d->Ho >= 1 && d->Wo >= 1))
        return false;
    const int lds = op == CKX_OP_CONV2D_FWD_I8 ? ckx::ConvStem<ckx::DT_I8>::lds_bytes(d->Wo) : ckx::ConvStem<ckx::DT_F16>::lds_bytes(d->Wo);
    return lds <= 160 * 1024;
}

// shapes the pointwise kernel covers: 1x1 filters without padding, a pixel of 256 or 512 bytes, output channels in
// whole blocks of 512
bool conv_pointwise_applicable(int op, const ckx_conv2d_desc* d, int epi)
{
    const int es      = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const bool epi_ok = op == CKX_OP_CONV2D_FWD_F16
                            ? (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_ADD_RELU)
                            : (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_REQUANT_CK || epi == CKX_EPI_REQUANT_RND ||
                               per_column_scale(epi));
    if(per_column_scale(epi) && d->C * es != 256) // (no registers for the scales beside the weights of a 512-byte pixel)
        return false;
    return (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && epi_ok && d->Y == 1 && d->X == 1 &&
           d->pad_top == 0 && d->pad_left == 0 && d->pad_bottom == 0 && d->pad_right == 0 &&
           (d->C * es == 256 || d->C * es == 512) && d->K >= 512 && d->K % 512 == 0 && d->N >= 1 && d->Ho >= 1 &&
           d->Wo >= 1;
}
// ... and the ones it is chosen for: enough pixels for every workgroup to amortise loading its weight slice
// (measured crossover against the best tile instance, C = 256, K = 512 / 1024: fp16 between 25 K and 50 K pixels
// per 512-channel block, int8 at about 12 K)
// (not for fp16 layers with 256-byte pixels that are plain GEMMs -- unit stride: C 128 -> K 512 at 28 x 28, N = 256, takes
// 72.8 us here and 56.5 on the dense GEMM kernels; with 512-byte pixels and in int8 the pointwise kernel stays ahead or
// level: fp16 C 256 -> K 1024 at 14 x 14 41.4 against 44.4, int8 24.2 against 32.9)
bool conv_is_dense_gemm(int op, const ckx_conv2d_desc* d);
bool conv_pointwise_preferred(int op, const ckx_conv2d_desc* d, int epi)
{
    const long px = (long)d->N * d->Ho * d->Wo * (d->K / 512);
    if(op == CKX_OP_CONV2D_FWD_F16 && d->C * 2 == 256 && conv_is_dense_gemm(op, d))
        return false;
    return conv_pointwise_applicable(op, d, epi) && px >= (op == CKX_OP_CONV2D_FWD_I8 ? 16 * 1024 : 40 * 1024);
}

// shapes the streaming 1x1 kernel covers: 1x1 filters, stride 1, no padding (the input is the [pixels, C] matrix), a pixel
// of 64 or 128 bytes with output channels in whole groups of 64 up to 256 or in whole blocks of 256, a pixel of 256 bytes
// with 64 or 128 output channels, one of 512 bytes with 64 (what a wave's registers hold of weights and pixel rows)
bool conv_rows_applicable(int op, const ckx_conv2d_desc* d, int epi)
{
    const int es      = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const bool epi_ok = op == CKX_OP_CONV2D_FWD_F16
                            ? (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_ADD_RELU)
                            : (epi == CKX_EPI_PASSTHROUGH || epi == CKX_EPI_REQUANT_CK || epi == CKX_EPI_REQUANT_RND);
    return (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && epi_ok && d->Y == 1 && d->X == 1 &&
           d->stride_h == 1 && d->stride_w == 1 && d->pad_top == 0 && d->pad_left == 0 && d->pad_bottom == 0 &&
           d->pad_right == 0 && (d->C * es == 64 || d->C * es == 128 || (d->C * es == 256 && d->K <= 128) || (d->C * es == 512 && d->K <= 64)) && d->K >= 64 &&
           d->K % 64 == 0 && (d->K <= 256 || d->K % 256 == 0) && d->N >= 1 && d->Ho == d->Hi && d->Wo == d->Wi && d->Ho >= 1 &&
           d->Wo >= 1;
}
// ... and the ones it is chosen for: enough rows for every wave of a full launch to run its two-deep pipeline, and few
// enough weight registers. Measured at N = 256 against the best tile instance: int8 C 64 -> K 64 at 56 x 56 19.6 against
// 37.6 us, C 64 -> K 256 64.7 against 84.0, C 256 -> K 64 42.0 against 47.0; fp16 C 64 -> K 64 33.2 against 34.5 (with
// bias + ReLU 33.4 against 38.8), C 256 -> K 64 99.2 against 104.9; but fp16 C 64 -> K 256 118 against 111, int8
// C 128 -> K 512 at 28 x 28 54.8 against 47.2 and int8 C 256 -> K 128 75.6 against 67.4 -- with 128 registers of weights half
// as many waves stream. The 256- and 512-byte pixels are left to the tile kernel altogether: level with its best instance
// at N = 256 (int8 C 256 -> K 64 43.5 against 42.5 on the 128 x 64 tile) and far behind at N = 32 (fp16 24.8 against
// 15.0 us: one row tile per iteration keeps too few bytes in flight when the launch is short).
bool conv_rows_preferred(int op, const ckx_conv2d_desc* d, int epi)
{
    const int px = d->C * (op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2);
    return conv_rows_applicable(op, d, epi) && (long)d->N * d->Ho * d->Wo >= 65536 &&
           (px == 64 || (px == 128 && d->K <= 128));
}

// A 1x1 filter with unit stride and no padding reads its input as the dense [pixels, C] matrix: past the specialists
// such a layer IS the GEMM out = in * wei^T, and it runs on the dense GEMM kernels -- no im2col address arithmetic per
// load, the four-wave body for the 256 x 256 tile -- through the GEMM family's own choice of instance and K runs.
// Measured at N = 256 against the im2col kernels on the ResNet-50 layers of this kind: fp16 C 1024 -> K 256 at 14 x 14 32.3
// -> 27.3 us, C 1024 -> K 512 56.4 -> 49.7, C 512 -> K 2048 at 7 x 7 36.9 -> 31.4; int8 C 2048 -> K 512 19.5 -> 17.3,
// C 256 -> K 128 at 56 x 56 68.4 -> 60.4; 2 - 16 % on all of them. (Above 128 pixels: below, the GEMM family's choice may be a
// skinny instance, which the conv instance list does not have.)
bool conv_is_dense_gemm(int op, const ckx_conv2d_desc* d)
{
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    return (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && d->Y == 1 && d->X == 1 && d->stride_h == 1 &&
           d->stride_w == 1 && d->pad_top == 0 && d->pad_left == 0 && d->pad_bottom == 0 && d->pad_right == 0 &&
           d->Ho == d->Hi && d->Wo == d->Wi && ((long)d->C * es) % 16 == 0 && (long)d->N * d->Ho * d->Wo > 128;
}

int check_conv(int op, const ckx_conv2d_desc* d, int epi, int instance)
{
    if(!d)
        return fail(CKX_INVALID_VALUE, "null conv descriptor");
    if(op != CKX_OP_CONV2D_FWD_I8 && op != CKX_OP_CONV2D_FWD_F16)
        return fail(CKX_INVALID_VALUE, "not a conv operator family");
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    if(instance != CKX_INSTANCE_AUTO && (instance < 0 || instance >= kNumConvInsts))
        return fail(CKX_INVALID_VALUE, "no such instance");
    if(epi < CKX_EPI_PASSTHROUGH || epi > CKX_EPI_RELU_MUL2_CLAMP || !epilogue_fits_dtype(es, epi) ||
       epi == CKX_EPI_CSHUFFLE_ADD_RELU)
        return fail(CKX_INVALID_VALUE, "epilogue not available for this operator");
    if(d->N < 0 || d->K < 0 || d->C < 0 || d->Hi <= 0 || d->Wi <= 0 || d->Y <= 0 || d->X <= 0 ||
       d->Ho < 0 || d->Wo < 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->dilation_h <= 0 ||
       d->dilation_w <= 0 || d->pad_top < 0 || d->pad_left < 0 || d->pad_bottom < 0 || d->pad_right < 0)
        return fail(CKX_INVALID_VALUE, "bad conv geometry");
    // window coordinates are kept as signed 16-bit pairs in the kernel: neither a window origin (ho * stride - pad,
    // lowest -pad, highest (Ho - 1) * stride - pad) nor origin + tap offset may leave [-32768, 32767]
    if(d->Hi > 16384 || d->Wi > 16384 || d->pad_top >= 16384 || d->pad_left >= 16384 ||
       (long)(d->Y - 1) * d->dilation_h >= 16384 || (long)(d->X - 1) * d->dilation_w >= 16384 ||
       (long)(d->Ho - 1) * d->stride_h - d->pad_top + (long)(d->Y - 1) * d->dilation_h >= 32768 ||
       (long)(d->Wo - 1) * d->stride_w - d->pad_left + (long)(d->X - 1) * d->dilation_w >= 32768)
        return fail(CKX_UNSUPPORTED, "spatial extents above 16384 (window coordinates above 32767) are not addressed");
    // the output extent has to be what the geometry implies (conv_util.cpp:103-114)
    const int ho = (d->Hi + d->pad_top + d->pad_bottom - ((d->Y - 1) * d->dilation_h + 1)) / d->stride_h + 1;
    const int wo = (d->Wi + d->pad_left + d->pad_right - ((d->X - 1) * d->dilation_w + 1)) / d->stride_w + 1;
    if(ho != d->Ho || wo != d->Wo)
        return fail(CKX_UNSUPPORTED, "output spatial lengths do not match the conv geometry");
    // a 16-byte vector along c must not cross a filter tap
    // (device_conv2d_fwd_xdl_nhwc_kyxc_nhwk.hpp:595-601)
    // (ConvolutionForwardSpecialization::OddC is the element-wise instance; AUTO sends such layers there)
    if(((long)d->C * es) % 16 && instance != CKX_INSTANCE_AUTO && instance != kConvGenericInstance && instance != kConvStemInstance)
        return fail(CKX_UNSUPPORTED, "C must be a multiple of 16 bytes for this instance (the element-wise instance and AUTO take any)");
    const long in_b  = (long)d->N * d->Hi * d->Wi * d->C * es;
    const long wei_b = (long)d->K * d->Y * d->X * d->C * es;
    const long out_b = (long)d->N * d->Ho * d->Wo * d->K * es;
    if(in_b >= (1l << 31) || wei_b >= (1l << 31) || out_b >= (1l << 31) ||
       (long)d->N * d->Ho * d->Wo >= (1l << 31))
        return fail(CKX_UNSUPPORTED, "tensors of 2 GiB or more are not addressed");
    if(instance == kConvPatchInstance && !conv_patch_applicable(op, d, epi))
        return fail(CKX_UNSUPPORTED, "the input-patch instance covers 3x3 stride-1 layers with C = K = 64, Wo = 56 or C = K = 128, Wo = 28 "
                                     "(the latter with PassThrough / requant / bias + ReLU epilogues)");
    if(instance == kConvStemInstance && !conv_stem_applicable(op, d, epi))
        return fail(CKX_UNSUPPORTED, "the stem instance covers 7x7 stride-2 layers with C = 3, K = 64 and padding 3, PassThrough / "
                                     "requant / bias + ReLU epilogues");
    if(instance == kConvPointwiseInstance && !conv_pointwise_applicable(op, d, epi))
        return fail(CKX_UNSUPPORTED, "the pointwise instance covers 1x1 layers without padding, C of 256 or 512 bytes, "
                                     "K a multiple of 512, PassThrough / requant / bias + ReLU epilogues");
    if(instance == kConvRowsInstance && !conv_rows_applicable(op, d, epi))
        return fail(CKX_UNSUPPORTED, "the streaming 1x1 instance covers 1x1 stride-1 layers without padding, C of 64 or 128 bytes with "
                                     "K a multiple of 64 up to 256 or a multiple of 256, C of 256 bytes with K = 64 / 128, C of 512 bytes "
                                     "with K = 64, PassThrough / requant / bias + ReLU epilogues");
    return CKX_OK;
}

long conv_workspace_bytes(int op, const ckx_conv2d_desc* d, int instance)
{
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const long M = (long)d->N * d->Ho * d->Wo;
    if(M <= 0 || d->K <= 0)
        return 0;
    if(instance == kConvPatchInstance || instance == kConvPointwiseInstance || instance == kConvGenericInstance ||
       instance == kConvStemInstance || instance == kConvRowsInstance || ((long)d->C * es) % 16 ||
       (instance == CKX_INSTANCE_AUTO &&
        (conv_patch_preferred(op, d, CKX_EPI_PASSTHROUGH) || conv_pointwise_preferred(op, d, CKX_EPI_PASSTHROUGH) ||
         conv_rows_preferred(op, d, CKX_EPI_PASSTHROUGH))))
        return 0;
    if(conv_is_dense_gemm(op, d))
        return gemm_workspace_bytes(es == 1 ? ckx::DT_I8 : ckx::DT_F16, (int)M, d->K, d->C, instance);
    const Plan pl = make_plan((int)M, d->K, d->Y * d->X * d->C * es, instance, 1l << 60, 0, false, true, d->Y * d->X);
    return pl.ksplit > 1 ? (long)pl.ksplit * M * d->K * 4 : 0;
}

int run_conv(int op, const void* in, const void* wei, void* out, const ckx_conv2d_desc* d, int epi, float sg,
             float sr, int instance, void* ws, long ws_bytes, void* stream, const DOperands& dops = DOperands{})
{
    int st = check_conv(op, d, epi, instance);
    if(st != CKX_OK)
        return st;
    if((st = check_d_operands(epi, d->K, dops)) != CKX_OK)
        return st;
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const int M = d->N * d->Ho * d->Wo, N = d->K, K = d->Y * d->X * d->C;
    if(M == 0 || N == 0)
        return CKX_OK;
    if(!in || !wei || !out)
        return fail(CKX_INVALID_VALUE, "null operand pointer");
    const bool misaligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(wei)) & 15) != 0;
    // (the stem kernel reads its operands element by element: alignment to the element size is all it asks of them; a bias
    // row means D0 stride 0)
    const bool stem_ok = conv_stem_applicable(op, d, epi) && dops.ldd0 == 0 &&
                         !((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(wei) | reinterpret_cast<uintptr_t>(out) |
                            reinterpret_cast<uintptr_t>(dops.d0)) & (es - 1));
    if(instance == kConvStemInstance || (instance == CKX_INSTANCE_AUTO && stem_ok))
    {
        if(!stem_ok)
            return fail(CKX_UNSUPPORTED, "the stem instance adds a bias row (D0 row stride 0) only and needs operands aligned to "
                                         "their element size");
        ckx::ConvStemArgs a;
        std::memset(&a, 0, sizeof(a));
        a.in = in, a.wei = wei, a.out = out, a.bias = dops.d0;
        a.N = d->N, a.Hi = d->Hi, a.Wi = d->Wi, a.Ho = d->Ho, a.Wo = d->Wo;
        a.epi = epi, a.scale_gemm = sg, a.scale_relu = sr;
        a.nt_store   = es == 1 && (long)M * N * es >= stream_output_bytes();
        hipError_t e = ckx::launch_conv_stem(es == 1 ? ckx::DT_I8 : ckx::DT_F16, a, (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kStemName);
    }
    if(instance == kConvGenericInstance || (instance == CKX_INSTANCE_AUTO && (misaligned || ((long)d->C * es) % 16)))
    {
        if((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(wei) | reinterpret_cast<uintptr_t>(out) |
            (f16_fused(epi) ? reinterpret_cast<uintptr_t>(dops.d0) | reinterpret_cast<uintptr_t>(dops.d1) : 0)) & (es - 1))
            return fail(CKX_UNSUPPORTED, "operands must be aligned to their element size");
        ckx::GemmArgs g;
        std::memset(&g, 0, sizeof(g));
        g.a = in, g.b = wei, g.c = out;
        g.M = M, g.N = N, g.K = K;
        g.ldb = K, g.ldc = N;
        g.epi = epi, g.scale_gemm = sg, g.scale_relu = sr;
        g.d0 = dops.d0, g.d1 = uses_d1(epi) ? dops.d1 : nullptr;
        g.ldd0 = dops.ldd0, g.ldd1 = dops.ldd1;
        g.ksplit  = 1;
        g.tiles_m = (M + 63) / 64, g.tiles_n = (N + 63) / 64;
        g.cv.Hi = d->Hi, g.cv.Wi = d->Wi, g.cv.C = d->C;
        g.cv.sH = d->stride_h, g.cv.sW = d->stride_w, g.cv.dH = d->dilation_h, g.cv.dW = d->dilation_w;
        g.cv.pT = d->pad_top, g.cv.pL = d->pad_left;
        g.cv.div_howo = make_magic((uint32_t)(d->Ho * d->Wo));
        g.cv.div_wo   = make_magic((uint32_t)d->Wo);
        g.cv.div_xc   = make_magic((uint32_t)(d->X * d->C));
        g.cv.div_c    = make_magic((uint32_t)d->C);
        ckx::GenericLayout lay{};
        lay.b_sn = K, lay.b_sk = 1;
        lay.X = d->X, lay.Y = d->Y;
        hipError_t e = ckx::launch_generic(es == 1 ? ckx::DT_I8 : ckx::DT_F16, 1, g, lay, (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kGenericName);
    }
    if(misaligned)
        return fail(CKX_UNSUPPORTED, "input and weight must be 16-byte aligned for this instance");
    if(ws && (reinterpret_cast<uintptr_t>(ws) & 15))
        return fail(CKX_INVALID_VALUE, "workspace must be 16-byte aligned");
    const bool patch_aligned = !((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(dops.d0) |
                                  (epi == CKX_EPI_ADD_RELU_ADD ? reinterpret_cast<uintptr_t>(dops.d1) : 0)) & 15);
    if(instance == kConvPatchInstance || (instance == CKX_INSTANCE_AUTO && conv_patch_preferred(op, d, epi) && patch_aligned))
    {
        if(!patch_aligned)
            return fail(CKX_UNSUPPORTED, "the input-patch instance needs 16-byte aligned output, bias and residual");
        ckx::ConvPatchArgs a;
        std::memset(&a, 0, sizeof(a));
        a.in = in, a.wei = wei, a.out = out;
        a.in_bytes  = (uint32_t)((long)d->N * d->Hi * d->Wi * d->C * es);
        a.wei_bytes = (uint32_t)((long)N * K * es);
        a.out_bytes = (uint32_t)((long)d->N * d->Ho * d->Wo * d->K * es);
        a.N = d->N, a.Hi = d->Hi, a.Wi = d->Wi, a.Ho = d->Ho, a.Wo = d->Wo;
        a.pT = d->pad_top, a.pL = d->pad_left;
        a.div_wo = make_magic((uint32_t)d->Wo);
        a.epi    = epi;
        a.bias = dops.d0, a.resi = epi == CKX_EPI_ADD_RELU_ADD ? dops.d1 : nullptr;
        a.scale_gemm = sg, a.scale_relu = sr;
        const bool fused = es == 1 ? per_column_scale(epi) : epi != CKX_EPI_PASSTHROUGH;
        hipError_t e     = d->C == 128 ? ckx::launch_conv_patch_wide(es == 1 ? ckx::DT_I8 : ckx::DT_F16, fused, a, (hipStream_t)stream)
                                       : ckx::launch_conv_patch(es == 1 ? ckx::DT_I8 : ckx::DT_F16, fused, a, (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kPatchName);
    }
    if(instance == kConvPointwiseInstance ||
       (instance == CKX_INSTANCE_AUTO && conv_pointwise_preferred(op, d, epi) && patch_aligned && dops.ldd0 == 0))
    {
        if(!patch_aligned)
            return fail(CKX_UNSUPPORTED, "the pointwise instance needs 16-byte aligned output and bias");
        if(epi == CKX_EPI_ADD_RELU && dops.ldd0 != 0)
            return fail(CKX_UNSUPPORTED, "the pointwise instance adds a bias row (D0 row stride 0) only");
        ckx::ConvPointwiseArgs a;
        std::memset(&a, 0, sizeof(a));
        a.in = in, a.wei = wei, a.out = out;
        a.in_bytes = (uint32_t)((long)d->N * d->Hi * d->Wi * d->C * es);
        a.M = M, a.Kout = N;
        a.Hi = d->Hi, a.Wi = d->Wi, a.Wo = d->Wo, a.HoWo = d->Ho * d->Wo, a.sH = d->stride_h, a.sW = d->stride_w;
        a.div_howo = make_magic((uint32_t)(d->Ho * d->Wo));
        a.div_wo   = make_magic((uint32_t)d->Wo);
        a.epi = epi, a.bias = dops.d0;
        a.scale_gemm = sg, a.scale_relu = sr;
        a.nt_store   = (long)M * N * es >= stream_output_bytes();
        hipError_t e = ckx::launch_conv_pointwise(es == 1 ? ckx::DT_I8 : ckx::DT_F16, d->C * es,
                                                  epi == CKX_EPI_ADD_RELU || per_column_scale(epi), a,
                                                  (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kPointwiseName);
    }
    if(instance == kConvRowsInstance ||
       (instance == CKX_INSTANCE_AUTO && conv_rows_preferred(op, d, epi) && patch_aligned && dops.ldd0 == 0))
    {
        if(!patch_aligned)
            return fail(CKX_UNSUPPORTED, "the streaming 1x1 instance needs 16-byte aligned output and bias");
        if(epi == CKX_EPI_ADD_RELU && dops.ldd0 != 0)
            return fail(CKX_UNSUPPORTED, "the streaming 1x1 instance adds a bias row (D0 row stride 0) only");
        ckx::ConvRowsArgs a;
        std::memset(&a, 0, sizeof(a));
        a.in = in, a.wei = wei, a.out = out, a.bias = dops.d0;
        a.in_bytes = (uint32_t)((long)M * d->C * es);
        a.M = M, a.C = d->C, a.Kout = N;
        a.epi = epi, a.scale_gemm = sg, a.scale_relu = sr;
        a.nt_store   = es == 1 && (long)M * N * es >= stream_output_bytes();
        hipError_t e = ckx::launch_conv_rows(es == 1 ? ckx::DT_I8 : ckx::DT_F16, d->C * es, epi == CKX_EPI_ADD_RELU, a,
                                             (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kRowsName);
    }
    if(conv_is_dense_gemm(op, d))
        return run_gemm(es == 1 ? ckx::DT_I8 : ckx::DT_F16, in, wei, out, M, N, K, K, K, N, CKX_ROW_MAJOR, CKX_COL_MAJOR,
                        CKX_ROW_MAJOR, epi, sg, sr, instance, ws, ws_bytes, stream, dops);
    const Plan pl = make_plan(M, N, K * es, instance, ws ? ws_bytes : 0, 0, false, true, d->Y * d->X, f16_fused(epi));
    const TileInstance& t = kTiles[pl.tile];
    ckx::GemmArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = in, g.b = wei, g.c = out;
    g.M = M, g.N = N, g.K = K;
    g.lda = 0, g.ldb = K, g.ldc = N;
    g.a_bytes    = (uint32_t)((long)d->N * d->Hi * d->Wi * d->C * es);
    g.b_bytes    = (uint32_t)((long)N * K * es);
    g.tiles_m    = (M + t.bm - 1) / t.bm;
    g.tiles_n    = (N + t.bn - 1) / t.bn;
    g.epi        = epi;
    g.scale_gemm = sg;
    g.scale_relu = sr;
    g.nt_store   = es == 1 && (long)M * N * es >= stream_output_bytes();
    g.d0 = dops.d0, g.d1 = uses_d1(epi) ? dops.d1 : nullptr;
    g.ldd0 = dops.ldd0, g.ldd1 = dops.ldd1;
    g.cv.Hi = d->Hi, g.cv.Wi = d->Wi, g.cv.C = d->C;
    g.cv.sH = d->stride_h, g.cv.sW = d->stride_w, g.cv.dH = d->dilation_h, g.cv.dW = d->dilation_w;
    g.cv.pT = d->pad_top, g.cv.pL = d->pad_left;
    g.cv.div_howo = make_magic((uint32_t)(d->Ho * d->Wo));
    g.cv.div_wo   = make_magic((uint32_t)d->Wo);
    g.cv.div_xc   = make_magic((uint32_t)(d->X * d->C));
    g.cv.div_c    = make_magic((uint32_t)d->C);
    g.ksplit = pl.ksplit;
    g.nk_per = pl.nk_per;
    g.ws     = ws;
    const bool fused = f16_fused(epi) && g.ksplit == 1;
    hipError_t e     = (es == 1  ? (per_column_scale(epi) && g.ksplit == 1 ? t.conv_i8_fused : t.conv_i8)
                        : fused ? t.conv_f16_fused
                                : t.conv_f16)(g, g.tiles_m * g.tiles_n * g.ksplit,
                                                                                 (hipStream_t)stream);
    if(e == hipSuccess && g.ksplit > 1)
        e = es == 1 ? launch_reduce<ckx::DT_I8>(g, (hipStream_t)stream)
                    : launch_reduce<ckx::DT_F16>(g, (hipStream_t)stream);
    if(e != hipSuccess)
        return hip_fail(e, t.name);
    return CKX_OK;
}

// ---------------------------------------------------------- conv forward, 1 / 2 / 3 spatial dimensions
// One and two dimensions are the 2-D problem (a 1-D conv is a 2-D conv on images one pixel high: same taps in
// the same order); so is a 3-D problem whose depth axis is not convolved (one tap, stride 1, no padding):
// N * D images.
bool convnd_as_2d(const ckx_convnd_desc* d, ckx_conv2d_desc& o)
{
    std::memset(&o, 0, sizeof(o));
    o.N = d->N, o.K = d->K, o.C = d->C;
    if(d->ndim == 1)
    {
        o.Hi = 1, o.Y = 1, o.Ho = 1, o.stride_h = 1, o.dilation_h = 1;
        o.Wi = d->in[0], o.X = d->filter[0], o.Wo = d->out[0], o.stride_w = d->stride[0];
        o.dilation_w = d->dilation[0], o.pad_left = d->pad_left[0], o.pad_right = d->pad_right[0];
        return true;
    }
    const int h = d->ndim - 2; // index of the H entries
    if(d->ndim == 3)
    {
        if(d->filter[0] != 1 || d->stride[0] != 1 || d->pad_left[0] != 0 || d->pad_right[0] != 0 ||
           d->in[0] != d->out[0] || d->in[0] <= 0 || (long)d->N * d->in[0] >= (1l << 31))
            return false;
        o.N = d->N * d->in[0];
    }
    o.Hi = d->in[h], o.Wi = d->in[h + 1], o.Y = d->filter[h], o.X = d->filter[h + 1];
    o.Ho = d->out[h], o.Wo = d->out[h + 1], o.stride_h = d->stride[h], o.stride_w = d->stride[h + 1];
    o.dilation_h = d->dilation[h], o.dilation_w = d->dilation[h + 1];
    o.pad_top = d->pad_left[h], o.pad_left = d->pad_left[h + 1];
    o.pad_bottom = d->pad_right[h], o.pad_right = d->pad_right[h + 1];
    return true;
}

int check_convnd(int op, const ckx_convnd_desc* d, int epi, int instance, ckx_conv2d_desc& as2d, bool& is2d)
{
    is2d = false;
    if(!d)
        return fail(CKX_INVALID_VALUE, "null conv descriptor");
    if(op != CKX_OP_CONV2D_FWD_I8 && op != CKX_OP_CONV2D_FWD_F16)
        return fail(CKX_INVALID_VALUE, "not a conv operator family");
    if(d->ndim < 1 || d->ndim > 3)
        return fail(CKX_INVALID_VALUE, "1, 2 or 3 spatial dimensions");
    if((is2d = convnd_as_2d(d, as2d)))
        return check_conv(op, &as2d, epi, instance);
    // three convolved dimensions: the tile instances
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    if(instance != CKX_INSTANCE_AUTO && (instance < 0 || instance >= kNumConvInsts))
        return fail(CKX_INVALID_VALUE, "no such instance");
    if(instance >= kNumTiles && instance != kConvGenericInstance)
        return fail(CKX_UNSUPPORTED, "the input-patch and pointwise instances cover two spatial dimensions");
    if(epi < CKX_EPI_PASSTHROUGH || epi > CKX_EPI_REQUANT_RND || !epilogue_fits_dtype(es, epi))
        return fail(CKX_INVALID_VALUE, "epilogue not available for this operator");
    if(d->N < 0 || d->K < 0 || d->C < 0)
        return fail(CKX_INVALID_VALUE, "bad conv geometry");
    long in_px = d->N, out_px = d->N, taps = 1;
    for(int i = 0; i < 3; ++i)
    {
        if(d->in[i] <= 0 || d->filter[i] <= 0 || d->out[i] < 0 || d->stride[i] <= 0 || d->dilation[i] <= 0 ||
           d->pad_left[i] < 0 || d->pad_right[i] < 0)
            return fail(CKX_INVALID_VALUE, "bad conv geometry");
        if(d->in[i] > 16384 || d->pad_left[i] >= 16384 || (long)(d->filter[i] - 1) * d->dilation[i] >= 16384 ||
           (long)(d->out[i] - 1) * d->stride[i] - d->pad_left[i] + (long)(d->filter[i] - 1) * d->dilation[i] >= 32768)
            return fail(CKX_UNSUPPORTED, "spatial extents above 16384 (window coordinates above 32767) are not addressed");
        // conv_util.cpp:103-114
        const int o = (d->in[i] + d->pad_left[i] + d->pad_right[i] - ((d->filter[i] - 1) * d->dilation[i] + 1)) /
                          d->stride[i] + 1;
        if(o != d->out[i])
            return fail(CKX_UNSUPPORTED, "output spatial lengths do not match the conv geometry");
        in_px *= d->in[i], out_px *= d->out[i], taps *= d->filter[i];
        if(in_px >= (1l << 31) || out_px >= (1l << 31) || taps >= (1l << 31))
            return fail(CKX_UNSUPPORTED, "tensors of 2 GiB or more are not addressed");
    }
    if(((long)d->C * es) % 16 && instance != CKX_INSTANCE_AUTO && instance != kConvGenericInstance)
        return fail(CKX_UNSUPPORTED, "C must be a multiple of 16 bytes for this instance (the element-wise instance and AUTO take any)");
    // (device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp:883-890 refuses tensors above 2 GB as well)
    if(in_px * d->C * es >= (1l << 31) || (long)d->K * taps * d->C * es >= (1l << 31) ||
       out_px * d->K * es >= (1l << 31) || taps * d->C >= (1l << 31))
        return fail(CKX_UNSUPPORTED, "tensors of 2 GiB or more are not addressed");
    return CKX_OK;
}

long convnd_workspace_bytes(int op, const ckx_convnd_desc* d, int instance)
{
    ckx_conv2d_desc d2;
    bool is2d;
    if(check_convnd(op, d, CKX_EPI_PASSTHROUGH, instance, d2, is2d) != CKX_OK)
        return 0;
    if(is2d)
        return conv_workspace_bytes(op, &d2, instance);
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const long M = (long)d->N * d->out[0] * d->out[1] * d->out[2];
    if(M <= 0 || d->K <= 0 || instance == kConvGenericInstance || ((long)d->C * es) % 16)
        return 0;
    const Plan pl = make_plan((int)M, d->K, d->filter[0] * d->filter[1] * d->filter[2] * d->C * es, instance, 1l << 60, 0, false, true);
    return pl.ksplit > 1 ? (long)pl.ksplit * M * d->K * 4 : 0;
}

int run_convnd(int op, const void* in, const void* wei, void* out, const ckx_convnd_desc* d, int epi, float sg,
               float sr, int instance, void* ws, long ws_bytes, void* stream)
{
    ckx_conv2d_desc d2;
    bool is2d;
    int st = check_convnd(op, d, epi, instance, d2, is2d);
    if(st != CKX_OK)
        return st;
    if(is2d)
        return run_conv(op, in, wei, out, &d2, epi, sg, sr, instance, ws, ws_bytes, stream);
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    const int M = d->N * d->out[0] * d->out[1] * d->out[2], N = d->K;
    const int K = d->filter[0] * d->filter[1] * d->filter[2] * d->C;
    if(M == 0 || N == 0)
        return CKX_OK;
    if(!in || !wei || !out)
        return fail(CKX_INVALID_VALUE, "null operand pointer");
    const bool misaligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(wei)) & 15) != 0;
    const bool generic =
        instance == kConvGenericInstance || (instance == CKX_INSTANCE_AUTO && (misaligned || ((long)d->C * es) % 16));
    if(misaligned && !generic)
        return fail(CKX_UNSUPPORTED, "input and weight must be 16-byte aligned for this instance");
    if(generic && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(wei) | reinterpret_cast<uintptr_t>(out)) & (es - 1)))
        return fail(CKX_UNSUPPORTED, "operands must be aligned to their element size");
    if(ws && (reinterpret_cast<uintptr_t>(ws) & 15))
        return fail(CKX_INVALID_VALUE, "workspace must be 16-byte aligned");
    const Plan pl         = generic ? Plan{} : make_plan(M, N, K * es, instance, ws ? ws_bytes : 0, 0, false, true);
    const TileInstance& t = kTiles[pl.tile];
    ckx::GemmArgs g;
    std::memset(&g, 0, sizeof(g));
    g.a = in, g.b = wei, g.c = out;
    g.M = M, g.N = N, g.K = K;
    g.lda = 0, g.ldb = K, g.ldc = N;
    g.a_bytes    = (uint32_t)((long)d->N * d->in[0] * d->in[1] * d->in[2] * d->C * es);
    g.b_bytes    = (uint32_t)((long)N * K * es);
    g.tiles_m    = (M + t.bm - 1) / t.bm;
    g.tiles_n    = (N + t.bn - 1) / t.bn;
    g.epi        = epi;
    g.scale_gemm = sg;
    g.scale_relu = sr;
    g.nt_store   = es == 1 && (long)M * N * es >= stream_output_bytes();
    g.cv.Di = d->in[0], g.cv.Hi = d->in[1], g.cv.Wi = d->in[2], g.cv.C = d->C;
    g.cv.sD = d->stride[0], g.cv.sH = d->stride[1], g.cv.sW = d->stride[2];
    g.cv.dD = d->dilation[0], g.cv.dH = d->dilation[1], g.cv.dW = d->dilation[2];
    g.cv.pF = d->pad_left[0], g.cv.pT = d->pad_left[1], g.cv.pL = d->pad_left[2];
    g.cv.div_dhowo = make_magic((uint32_t)(d->out[0] * d->out[1] * d->out[2]));
    g.cv.div_howo  = make_magic((uint32_t)(d->out[1] * d->out[2]));
    g.cv.div_wo    = make_magic((uint32_t)d->out[2]);
    g.cv.div_yxc   = make_magic((uint32_t)(d->filter[1] * d->filter[2] * d->C));
    g.cv.div_xc    = make_magic((uint32_t)(d->filter[2] * d->C));
    g.cv.div_c     = make_magic((uint32_t)d->C);
    g.ksplit = pl.ksplit;
    g.nk_per = pl.nk_per;
    g.ws     = ws;
    if(generic)
    {
        g.tiles_m = (M + 63) / 64, g.tiles_n = (N + 63) / 64;
        g.ksplit  = 1;
        ckx::GenericLayout lay{};
        lay.b_sn = K, lay.b_sk = 1;
        lay.X = d->filter[2], lay.Y = d->filter[1];
        hipError_t e = ckx::launch_generic(es == 1 ? ckx::DT_I8 : ckx::DT_F16, 2, g, lay, (hipStream_t)stream);
        return e == hipSuccess ? CKX_OK : hip_fail(e, kGenericName);
    }
    const tile_launch_fn launch = ckx::conv3d_tile(es == 1 ? ckx::DT_I8 : ckx::DT_F16, pl.tile);
    if(!launch)
        return fail(CKX_UNSUPPORTED, "no kernel variant for this instance");
    hipError_t e = launch(g, g.tiles_m * g.tiles_n * g.ksplit, (hipStream_t)stream);
    if(e == hipSuccess && g.ksplit > 1)
        e = es == 1 ? launch_reduce<ckx::DT_I8>(g, (hipStream_t)stream) : launch_reduce<ckx::DT_F16>(g, (hipStream_t)stream);
    if(e != hipSuccess)
        return hip_fail(e, t.name);
    return CKX_OK;
}

} // namespace

extern "C" {

const char* ckx_version(void) { return "ckx-mi355 0.1 (gfx950)"; }
const char* ckx_last_error(void) { return g_last_error.c_str(); }

int ckx_num_instances(int op)
{
    if(op == CKX_OP_GEMM_I8 || op == CKX_OP_GEMM_F16 || op == CKX_OP_GEMM_BF16)
        return kNumGemmInsts;
    if(op == CKX_OP_GEMM_SPLITK)
        return kNumTiles;
    if(op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8)
        return kNumConvInsts; // + the input-patch, the pointwise, the stem, the streaming 1x1 and the element-wise kernel
    if(op == CKX_OP_BATCHED_GEMM_GEMM || op == CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM)
        return ckx::kNumGemmGemmInstances;
    return 0;
}

const char* ckx_instance_name(int op, int instance)
{
    static thread_local std::string s;
    const char* fam = family_prefix(op);
    if(!fam || instance < 0 || instance >= ckx_num_instances(op))
        return nullptr;
    s = std::string(fam) + "<" +
        (op == CKX_OP_BATCHED_GEMM_GEMM || op == CKX_OP_BATCHED_GEMM_SOFTMAX_GEMM
             ? ckx::gemm_gemm_instance_name(instance)
         : (op == CKX_OP_CONV2D_FWD_F16 || op == CKX_OP_CONV2D_FWD_I8) && instance >= kNumTiles
             ? (instance == kConvPatchInstance ? kPatchName : instance == kConvPointwiseInstance ? kPointwiseName
                : instance == kConvStemInstance ? kStemName : instance == kConvRowsInstance ? kRowsName : kGenericName)
             : instance == kGenericGemmInstance ? kGenericName
             : instance >= kNumTiles            ? kSkinny[instance - kNumTiles].name
                                                : kTiles[instance].name) +
        ">";
    return s.c_str();
}

int ckx_gemm_i8_is_supported(int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sc, int al,
                             int bl, int cl, int epilogue, int instance)
{
    if(per_column_scale(epilogue))
        return fail(CKX_UNSUPPORTED, "epilogues with a scale row as D operand go through ckx_gemm_i8_multiple_d");
    return check_gemm_shape(ckx::DT_I8, M, N, K, sa, sb, sc, al, bl, cl, epilogue, instance);
}

int64_t ckx_gemm_i8_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance)
{
    return gemm_workspace_bytes(ckx::DT_I8, M, N, K, instance);
}

int ckx_gemm_i8(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                int32_t sb, int32_t sc, int al, int bl, int cl, int epilogue, float scale_gemm,
                float scale_relu, int instance, void* workspace, int64_t workspace_bytes, void* stream)
{
    return run_gemm(ckx::DT_I8, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, epilogue, scale_gemm, scale_relu,
                    instance, workspace, workspace_bytes, stream);
}

int ckx_set_big_tile_waves(int waves)
{
    const int before = big_tile_waves();
    g_big_tile_waves.store((waves == 4 || waves == 8) ? waves : 0, std::memory_order_relaxed);
    return before;
}

int ckx_set_forced_k_runs(int k_runs)
{
    const int before = force_ksplit();
    g_force_ksplit.store(k_runs < 0 ? 0 : k_runs, std::memory_order_relaxed);
    return before;
}

int ckx_gemm_plan(int op, int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sc, int al, int bl, int cl,
                  int epilogue, int32_t batch, int64_t workspace_bytes, int* instance, int* k_runs)
{
    if(op != CKX_OP_GEMM_I8 && op != CKX_OP_GEMM_F16 && op != CKX_OP_GEMM_BF16)
        return fail(CKX_INVALID_VALUE, "not a GEMM operator family");
    if(!instance || !k_runs || batch < 1)
        return fail(CKX_INVALID_VALUE, "bad plan query");
    const int dt = op == CKX_OP_GEMM_I8 ? ckx::DT_I8 : op == CKX_OP_GEMM_BF16 ? ckx::DT_BF16 : ckx::DT_F16;
    int st       = check_gemm_shape(dt, M, N, K, sa, sb, sc, al, bl, cl, epilogue, *instance);
    if(st != CKX_OK)
        return st;
    const bool ta = al == CKX_COL_MAJOR, tb = bl == CKX_ROW_MAJOR;
    if(*instance == kGenericGemmInstance ||
       (*instance == CKX_INSTANCE_AUTO && gemm_needs_generic(dt, M, N, K, sa, sb, ta, tb, epilogue)))
    {
        *instance = kGenericGemmInstance, *k_runs = 1;
        return CKX_OK;
    }
    const GemmChoice ch = choose_gemm(dt, M, N, K, ta || tb, *instance, workspace_bytes > 0 ? workspace_bytes : 0, 0, batch);
    *instance = ch.instance, *k_runs = ch.ksplit;
    return CKX_OK;
}

int ckx_conv2d_fwd_plan(int op, const ckx_conv2d_desc* d, int epilogue, int64_t workspace_bytes, int* instance, int* k_runs)
{
    if(!instance || !k_runs)
        return fail(CKX_INVALID_VALUE, "bad plan query");
    int st = check_conv(op, d, epilogue, *instance);
    if(st != CKX_OK)
        return st;
    const int es = op == CKX_OP_CONV2D_FWD_I8 ? 1 : 2;
    *k_runs      = 1;
    if(*instance == CKX_INSTANCE_AUTO)
    {
        if(conv_stem_applicable(op, d, epilogue))
            *instance = kConvStemInstance;
        else if(((long)d->C * es) % 16)
            *instance = kConvGenericInstance;
        else if(conv_patch_preferred(op, d, epilogue))
            *instance = kConvPatchInstance;
        else if(conv_pointwise_preferred(op, d, epilogue))
            *instance = kConvPointwiseInstance;
        else if(conv_rows_preferred(op, d, epilogue))
            *instance = kConvRowsInstance;
    }
    if((*instance == CKX_INSTANCE_AUTO || *instance < kNumTiles) && conv_is_dense_gemm(op, d))
    {
        const GemmChoice ch = choose_gemm(es == 1 ? ckx::DT_I8 : ckx::DT_F16, d->N * d->Ho * d->Wo, d->K, d->C, false, *instance,
                                          workspace_bytes > 0 ? workspace_bytes : 0, 0, 1);
        *instance = ch.instance, *k_runs = ch.ksplit;
    }
    else if(*instance == CKX_INSTANCE_AUTO || *instance < kNumTiles)
    {
        const Plan pl = make_plan((long)d->N * d->Ho * d->Wo, d->K, d->Y * d->X * d->C * es, *instance,
                                  workspace_bytes > 0 ? workspace_bytes : 0, 0, false, true, d->Y * d->X,
                                  f16_fused(epilogue));
        *instance = pl.tile, *k_runs = pl.ksplit;
    }
    return CKX_OK;
}

int ckx_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sc, int al,
                              int bl, int cl, int instance)
{
    return check_gemm_shape(ckx::DT_F16, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, instance);
}

int64_t ckx_gemm_f16_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance)
{
    return gemm_workspace_bytes(ckx::DT_F16, M, N, K, instance);
}

int ckx_gemm_f16(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                 int32_t sb, int32_t sc, int al, int bl, int cl, int instance, void* workspace,
                 int64_t workspace_bytes, void* stream)
{
    return run_gemm(ckx::DT_F16, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, 1.0f, 1.0f,
                    instance, workspace, workspace_bytes, stream);
}

int64_t ckx_gemm_splitk_workspace_bytes(int op, int32_t M, int32_t N, int32_t K, int32_t k_batch)
{
    if((op != CKX_OP_GEMM_I8 && op != CKX_OP_GEMM_F16) || M <= 0 || N <= 0 || K < 0 || k_batch < 1)
        return 0;
    const int runs = splitk_runs(K * (op == CKX_OP_GEMM_I8 ? 1 : 2), k_batch);
    return runs > 1 ? (int64_t)runs * M * N * 4 : 0;
}

int ckx_gemm_i8_splitk(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                       int32_t sb, int32_t sc, int al, int bl, int cl, int epilogue, float scale_gemm,
                       float scale_relu, int instance, int32_t k_batch, void* workspace, int64_t workspace_bytes,
                       void* stream)
{
    if(k_batch < 1)
        return fail(CKX_INVALID_VALUE, "KBatch must be at least 1");
    return run_gemm(ckx::DT_I8, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, epilogue, scale_gemm, scale_relu,
                    instance, workspace, workspace_bytes, stream, DOperands{}, k_batch);
}

int ckx_gemm_i8_splitk_noalloc(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                               int32_t sb, int32_t sc, int al, int bl, int cl, int epilogue, float scale_gemm,
                               float scale_relu, int instance, int32_t k_batch, void* stream)
{
    if(k_batch < 1)
        return fail(CKX_INVALID_VALUE, "KBatch must be at least 1");
    // (argument errors and empty problems are answered before the GPU is touched)
    if(int st = check_gemm_shape(ckx::DT_I8, M, N, K, sa, sb, sc, al, bl, cl, epilogue, instance))
        return st;
    if(k_batch > 8)
        return fail(CKX_UNSUPPORTED, "KBatch must be 1..8");
    if(M == 0 || N == 0)
        return CKX_OK;
    const int64_t need = ckx_gemm_splitk_workspace_bytes(CKX_OP_GEMM_I8, M, N, K, k_batch);
    if(need > (int64_t)CKX_STATIC_WORKSPACE_BYTES)
        return fail(CKX_UNSUPPORTED, "this split needs " + std::to_string(need) +
                                         " bytes of workspace, the library's static workspace holds " +
                                         std::to_string((long)CKX_STATIC_WORKSPACE_BYTES) +
                                         ": use ckx_gemm_i8_splitk with a workspace of the caller's");
    void* ws = nullptr;
    if(int st = static_workspace(&ws))
        return st;
    return run_gemm(ckx::DT_I8, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, epilogue, scale_gemm, scale_relu,
                    instance, ws, (long)CKX_STATIC_WORKSPACE_BYTES, stream, DOperands{}, k_batch);
}

int ckx_gemm_f16_splitk(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                        int32_t sb, int32_t sc, int al, int bl, int cl, int instance, int32_t k_batch,
                        void* workspace, int64_t workspace_bytes, void* stream)
{
    if(k_batch < 1)
        return fail(CKX_INVALID_VALUE, "KBatch must be at least 1");
    return run_gemm(ckx::DT_F16, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, 1.0f, 1.0f,
                    instance, workspace, workspace_bytes, stream, DOperands{}, k_batch);
}

int ckx_gemm_bf16_is_supported(int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sc, int al,
                               int bl, int cl, int instance)
{
    return check_gemm_shape(ckx::DT_BF16, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, instance);
}

int64_t ckx_gemm_bf16_workspace_bytes(int32_t M, int32_t N, int32_t K, int instance)
{
    return gemm_workspace_bytes(ckx::DT_BF16, M, N, K, instance);
}

int ckx_gemm_bf16(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                  int32_t sb, int32_t sc, int al, int bl, int cl, int instance, void* workspace,
                  int64_t workspace_bytes, void* stream)
{
    return run_gemm(ckx::DT_BF16, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, 1.0f, 1.0f,
                    instance, workspace, workspace_bytes, stream);
}

int ckx_batched_gemm_is_supported(int op, int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sc,
                                  int64_t bsa, int64_t bsb, int64_t bsc, int32_t batch, int al, int bl, int cl,
                                  int epilogue, int instance)
{
    if(op != CKX_OP_GEMM_I8 && op != CKX_OP_GEMM_F16)
        return fail(CKX_INVALID_VALUE, "not a GEMM operator family");
    const int dt = op == CKX_OP_GEMM_I8 ? ckx::DT_I8 : ckx::DT_F16;
    int st       = check_gemm_shape(dt, M, N, K, sa, sb, sc, al, bl, cl, epilogue, instance);
    return st != CKX_OK ? st : check_batch(dt, M, N, K, sa, sb, sc, al == CKX_COL_MAJOR, bl == CKX_ROW_MAJOR, epilogue, instance, 0, batch,
                                         bsa, bsb, bsc);
}

int ckx_batched_gemm_i8(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                        int32_t sb, int32_t sc, int64_t bsa, int64_t bsb, int64_t bsc, int32_t batch, int al, int bl,
                        int cl, int epilogue, float scale_gemm, float scale_relu, int instance, void* stream)
{
    return run_gemm(ckx::DT_I8, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, epilogue, scale_gemm, scale_relu,
                    instance, nullptr, 0, stream, DOperands{}, 0, batch, bsa, bsb, bsc);
}

int ckx_batched_gemm_f16(const void* a, const void* b, void* c, int32_t M, int32_t N, int32_t K, int32_t sa,
                         int32_t sb, int32_t sc, int64_t bsa, int64_t bsb, int64_t bsc, int32_t batch, int al, int bl,
                         int cl, int instance, void* stream)
{
    return run_gemm(ckx::DT_F16, a, b, c, M, N, K, sa, sb, sc, al, bl, cl, CKX_EPI_PASSTHROUGH, 1.0f, 1.0f,
                    instance, nullptr, 0, stream, DOperands{}, 0, batch, bsa, bsb, bsc);
}

int ckx_gemm_f16_multiple_d_is_supported(int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sd0,
                                         int32_t sd1, int32_t se, int al, int bl, int el, int cde_op, int instance)
{
    if(!f16_fused(cde_op))
        return fail(CKX_INVALID_VALUE, "not a CDE element-wise operation");
    int st = check_gemm_shape(ckx::DT_F16, M, N, K, sa, sb, se, al, bl, el, cde_op, instance);
    if(st != CKX_OK)
        return st;
    DOperands d;
    d.d0 = d.d1 = &d; // only the strides are under test here
    d.ldd0 = sd0, d.ldd1 = sd1;
    return check_d_operands(cde_op, N, d);
}

int ckx_gemm_f16_multiple_d(const void* a, const void* b, const void* d0, const void* d1, void* e, int32_t M,
                            int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sd0, int32_t sd1, int32_t se,
                            int al, int bl, int el, int cde_op, int instance, void* workspace,
                            int64_t workspace_bytes, void* stream)
{
    if(!f16_cde_op(cde_op))
        return fail(CKX_INVALID_VALUE, "not a CDE element-wise operation");
    DOperands d;
    d.d0 = d0, d.d1 = d1, d.ldd0 = sd0, d.ldd1 = sd1;
    return run_gemm(ckx::DT_F16, a, b, e, M, N, K, sa, sb, se, al, bl, el, cde_op, 1.0f, 1.0f, instance, workspace,
                    workspace_bytes, stream, d);
}

int ckx_gemm_f16_bilinear(const void* a, const void* b, const void* d0, void* e, int32_t M, int32_t N, int32_t K,
                          int32_t sa, int32_t sb, int32_t sd, int32_t se, int al, int bl, int el, float alpha,
                          float beta, int instance, void* workspace, int64_t workspace_bytes, void* stream)
{
    DOperands d;
    d.d0 = d0, d.ldd0 = sd;
    return run_gemm(ckx::DT_F16, a, b, e, M, N, K, sa, sb, se, al, bl, el, CKX_EPI_BILINEAR, alpha, beta, instance,
                    workspace, workspace_bytes, stream, d);
}

int ckx_gemm_i8_multiple_d_is_supported(int32_t M, int32_t N, int32_t K, int32_t sa, int32_t sb, int32_t sd0,
                                        int32_t se, int al, int bl, int el, int cde_op, int instance)
{
    if(!per_column_scale(cde_op))
        return fail(CKX_INVALID_VALUE, "not a CDE element-wise operation of the int8 family");
    int st = check_gemm_shape(ckx::DT_I8, M, N, K, sa, sb, se, al, bl, el, cde_op, instance);
    if(st != CKX_OK)
        return st;
    static const float probe = 0.0f; // only the stride is under test here
    DOperands d;
    d.d0 = &probe, d.ldd0 = sd0;
    return check_d_operands(cde_op, N, d);
}

int ckx_gemm_i8_multiple_d(const void* a, const void* b, const void* d0, void* e, int32_t M, int32_t N, int32_t K,
                           int32_t sa, int32_t sb, int32_t sd0, int32_t se, int al, int bl, int el, int cde_op,
                           int instance, void* workspace, int64_t workspace_bytes, void* stream)
{
    if(!per_column_scale(cde_op))
        return fail(CKX_INVALID_VALUE, "not a CDE element-wise operation of the int8 family");
    DOperands d;
    d.d0 = d0, d.ldd0 = sd0;
    return run_gemm(ckx::DT_I8, a, b, e, M, N, K, sa, sb, se, al, bl, el, cde_op, 1.0f, 1.0f, instance, workspace,
                    workspace_bytes, stream, d);
}

int ckx_conv2d_fwd_i8_multiple_d(const void* in, const void* wei, const void* scale, void* out,
                                 const ckx_conv2d_desc* desc, int out_op, int instance, void* workspace,
                                 int64_t workspace_bytes, void* stream)
{
    if(!per_column_scale(out_op))
        return fail(CKX_INVALID_VALUE, "not a per-channel requant output operation");
    DOperands d;
    d.d0 = scale, d.ldd0 = 0;
    return run_conv(CKX_OP_CONV2D_FWD_I8, in, wei, out, desc, out_op, 1.0f, 1.0f, instance, workspace,
                    workspace_bytes, stream, d);
}

int ckx_conv2d_fwd_bias_activation_f16(const void* in, const void* wei, void* out, const void* bias,
                                       const void* resi, const ckx_conv2d_desc* desc, int out_op, int instance,
                                       void* workspace, int64_t workspace_bytes, void* stream)
{
    if(out_op != CKX_EPI_ADD_RELU && out_op != CKX_EPI_ADD_RELU_ADD)
        return fail(CKX_INVALID_VALUE, "not a bias-activation output operation");
    DOperands d;
    d.d0 = bias, d.ldd0 = 0;
    d.d1 = resi, d.ldd1 = desc ? desc->K : 0;
    return run_conv(CKX_OP_CONV2D_FWD_F16, in, wei, out, desc, out_op, 1.0f, 1.0f, instance, workspace,
                    workspace_bytes, stream, d);
}

int ckx_conv2d_fwd_is_supported(int op, const ckx_conv2d_desc* desc, int epilogue, int instance)
{
    return check_conv(op, desc, epilogue, instance);
}

int64_t ckx_conv2d_fwd_workspace_bytes(int op, const ckx_conv2d_desc* desc, int instance)
{
    if(check_conv(op, desc, CKX_EPI_PASSTHROUGH, instance) != CKX_OK)
        return 0;
    return conv_workspace_bytes(op, desc, instance);
}

int ckx_conv2d_fwd_i8(const void* in, const void* wei, void* out, const ckx_conv2d_desc* desc, int epilogue,
                      float scale_gemm, float scale_relu, int instance, void* workspace, int64_t workspace_bytes,
                      void* stream)
{
    return run_conv(CKX_OP_CONV2D_FWD_I8, in, wei, out, desc, epilogue, scale_gemm, scale_relu, instance,
                    workspace, workspace_bytes, stream);
}

int ckx_conv2d_fwd_f16(const void* in, const void* wei, void* out, const ckx_conv2d_desc* desc, int instance,
                       void* workspace, int64_t workspace_bytes, void* stream)
{
    return run_conv(CKX_OP_CONV2D_FWD_F16, in, wei, out, desc, CKX_EPI_PASSTHROUGH, 1.0f, 1.0f, instance,
                    workspace, workspace_bytes, stream);
}

int ckx_convnd_fwd_is_supported(int op, const ckx_convnd_desc* desc, int epilogue, int instance)
{
    ckx_conv2d_desc d2;
    bool is2d;
    return check_convnd(op, desc, epilogue, instance, d2, is2d);
}

int64_t ckx_convnd_fwd_workspace_bytes(int op, const ckx_convnd_desc* desc, int instance)
{
    return convnd_workspace_bytes(op, desc, instance);
}

int ckx_convnd_fwd(int op, const void* in, const void* wei, void* out, const ckx_convnd_desc* desc, int epilogue,
                   float scale_gemm, float scale_relu, int instance, void* workspace, int64_t workspace_bytes,
                   void* stream)
{
    return run_convnd(op, in, wei, out, desc, epilogue, scale_gemm, scale_relu, instance, workspace, workspace_bytes,
                      stream);
}

int ckx_batched_gemm_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t O, int32_t batch,
                                           int32_t sa, int32_t sb0, int32_t sb1, int32_t sc, int64_t bsa,
                                           int64_t bsb0, int64_t bsb1, int64_t bsc, int instance)
{
    std::string why;
    if(!ckx::gemm_gemm_supported(M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc, instance, why))
        return fail(why.rfind("invalid", 0) == 0 ? CKX_INVALID_VALUE : CKX_UNSUPPORTED, why);
    return CKX_OK;
}

int ckx_batched_gemm_gemm_f16(const void* a, const void* b0, const void* b1, void* c, int32_t M, int32_t N,
                              int32_t K, int32_t O, int32_t batch, int32_t sa, int32_t sb0, int32_t sb1,
                              int32_t sc, int64_t bsa, int64_t bsb0, int64_t bsb1, int64_t bsc, int instance,
                              void* stream)
{
    int st = ckx_batched_gemm_gemm_f16_is_supported(M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc,
                                                    instance);
    if(st != CKX_OK)
        return st;
    if(M == 0 || O == 0 || batch == 0)
        return CKX_OK;
    if(!a || !c || (N > 0 && (!b0 || !b1))) // (N == 0: B0 and B1 are empty, C = 0)
        return fail(CKX_INVALID_VALUE, "null operand pointer");
    if((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b0) | reinterpret_cast<uintptr_t>(b1) |
        reinterpret_cast<uintptr_t>(c)) & 15)
        return fail(CKX_UNSUPPORTED, "operands must be 16-byte aligned");
    hipError_t e = ckx::gemm_gemm_launch(a, b0, b1, c, M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc,
                                         instance, (hipStream_t)stream);
    if(e != hipSuccess)
        return hip_fail(e, "batched_gemm_gemm");
    return CKX_OK;
}

int ckx_batched_gemm_softmax_gemm_f16_is_supported(int32_t M, int32_t N, int32_t K, int32_t O, int32_t batch,
                                                   int32_t sa, int32_t sb0, int32_t sb1, int32_t sc, int64_t bsa,
                                                   int64_t bsb0, int64_t bsb1, int64_t bsc, float acc0_scale,
                                                   int mask_out_upper_triangle, int instance)
{
    if(!(acc0_scale == acc0_scale) || acc0_scale - acc0_scale != 0.0f)
        return fail(CKX_INVALID_VALUE, "the score scale must be finite");
    if(mask_out_upper_triangle != 0 && mask_out_upper_triangle != 1)
        return fail(CKX_INVALID_VALUE, "mask_out_upper_triangle is 0 or 1");
    return ckx_batched_gemm_gemm_f16_is_supported(M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc, instance);
}

int ckx_batched_gemm_softmax_gemm_f16(const void* a, const void* b0, const void* b1, void* c, int32_t M, int32_t N,
                                      int32_t K, int32_t O, int32_t batch, int32_t sa, int32_t sb0, int32_t sb1,
                                      int32_t sc, int64_t bsa, int64_t bsb0, int64_t bsb1, int64_t bsc,
                                      float acc0_scale, int mask_out_upper_triangle, int instance, void* stream)
{
    int st = ckx_batched_gemm_softmax_gemm_f16_is_supported(M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc,
                                                            acc0_scale, mask_out_upper_triangle, instance);
    if(st != CKX_OK)
        return st;
    if(M == 0 || O == 0 || batch == 0)
        return CKX_OK;
    if(!a || !c || (N > 0 && (!b0 || !b1))) // (N == 0: B0 and B1 are empty, C = 0)
        return fail(CKX_INVALID_VALUE, "null operand pointer");
    if((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b0) | reinterpret_cast<uintptr_t>(b1) |
        reinterpret_cast<uintptr_t>(c)) & 15)
        return fail(CKX_UNSUPPORTED, "operands must be 16-byte aligned");
    hipError_t e = ckx::gemm_gemm_launch(a, b0, b1, c, M, N, K, O, batch, sa, sb0, sb1, sc, bsa, bsb0, bsb1, bsc,
                                         instance, (hipStream_t)stream, true, acc0_scale, mask_out_upper_triangle != 0);
    if(e != hipSuccess)
        return hip_fail(e, "batched_gemm_softmax_gemm");
    return CKX_OK;
}

int ckx_time_launches(ckx_launch_fn fn, void* user, int n_warmup, int n_repeat, void* stream, float* ms)
{
    if(!fn || !ms || n_repeat <= 0 || n_warmup < 0)
        return fail(CKX_INVALID_VALUE, "bad timing request");
    hipStream_t s = (hipStream_t)stream;
    for(int i = 0; i < n_warmup; ++i)
        if(int r = fn(user))
            return r;
    hipEvent_t e0, e1;
    hipError_t e = hipEventCreate(&e0);
    if(e != hipSuccess)
        return hip_fail(e, "hipEventCreate");
    e = hipEventCreate(&e1);
    if(e != hipSuccess)
    {
        (void)hipEventDestroy(e0);
        return hip_fail(e, "hipEventCreate");
    }
    int rc = CKX_OK;
    e      = hipStreamSynchronize(s);
    if(e == hipSuccess)
        e = hipEventRecord(e0, s);
    for(int i = 0; i < n_repeat && e == hipSuccess && rc == CKX_OK; ++i)
        rc = fn(user);
    if(e == hipSuccess)
        e = hipEventRecord(e1, s);
    if(e == hipSuccess)
        e = hipEventSynchronize(e1);
    float total = 0;
    if(e == hipSuccess)
        e = hipEventElapsedTime(&total, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if(e != hipSuccess)
        return hip_fail(e, "ckx_time_launches");
    *ms = total / (float)n_repeat;
    return rc;
}

} // extern "C"
