// K1 / K4: int8 x int8 -> int32 tiled GEMM on the gfx950 matrix cores with the offset contribution and the
// output stage fused into the epilogue, and an implicit-GEMM (on-the-fly im2col) variant of the A loader.
//
// What it replaces in the reference (all O(M*N*K) work of the path plus both O(M*N) passes):
//   arm_gemm int8 kernels behind CpuGemmAssemblyDispatch (src/cpu/operators/internal/CpuGemmAssemblyDispatch.cpp:640-838)
//   or CpuGemmLowpMatrixMultiplyKernel (src/cpu/kernels/CpuGemmLowpMatrixMultiplyKernel.cpp:722-883),
//   CpuGemmLowpOffsetContribution{,OutputStage}Kernel (src/cpu/kernels/CpuGemmLowpOffsetContributionOutputStageKernel.cpp:248-461),
//   CpuConvertQuantizedSignednessKernel (x ^ 0x80 folded into the loader), and for the conv loader
//   CpuIm2ColKernel (src/cpu/kernels/directconv2d/impl.h:148-220,307-389).
//
// Data layout: A row-major [M][lda] int8 (K contiguous, rows 4-byte aligned; 16-byte loads), B pre-packed as Bp[Np][Kp] int8
// (K contiguous, zero padded) so both operands are staged the same way. A block computes a BM x BN tile; per
// K step it stages BM x BK of A and BN x BK of B in LDS (two stages), 16 bytes per lane per access, with an XOR swizzle
// of the 16-byte column index so that both the staging writes and the operand reads are bank-conflict free.
// Each wave owns a (BM/WM) x (BN/WN) sub-tile as 32x32 accumulator blocks fed by v_mfma_i32_32x32x32_i8.
#include "mfma_common.hpp"

namespace mi355
{
template <int BM, int BN, int BK, int WM, int WN, int EPI, bool FLIP_A, bool CONV>
__global__ __launch_bounds__(WM *WN * 64) void gemm_mfma_kernel(GemmArgs g)
{
    constexpr int NT       = WM * WN * 64;
    constexpr int CPR      = BK / 16;
    constexpr int A_CHUNKS = BM * CPR / NT;
    constexpr int B_CHUNKS = BN * CPR / NT;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 32, FN = TN / 32;
    constexpr int STAGE = (BM + BN) * BK;
    static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "loader shape");
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile");

    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    int tm, tn;
    tile_coords(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int bz = blockIdx.z;

    const int8_t *__restrict__ A  = g.A + (int64_t)bz * g.a_batch_stride;
    const int8_t *__restrict__ Bp = g.Bp + (int64_t)bz * g.bp_batch_stride + (int64_t)n0 * g.Kp;

    // per-thread staging assignment (fixed for the whole K loop)
    int     a_lds[A_CHUNKS], b_lds[B_CHUNKS];
    int64_t a_off[A_CHUNKS]; // dense: byte offset of (row, col*16) ; conv: byte offset of image n
    int     a_iy0[A_CHUNKS], a_ix0[A_CHUNKS];
    int     a_col[A_CHUNKS];
    int64_t b_off[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i)
    {
        const int c   = tid + i * NT;
        const int row = c / CPR, col = c % CPR;
        a_lds[i]      = row * BK + ((col ^ swz<CPR>(row)) << 4);
        a_col[i]      = col * 16;
        const int gr  = min(m0 + row, g.M - 1);
        if (CONV)
        {
            const int ox = gr % g.conv.OW;
            const int t  = gr / g.conv.OW;
            const int oy = t % g.conv.OH;
            const int n  = t / g.conv.OH;
            a_off[i]     = (int64_t)n * g.conv.H * g.conv.W * g.conv.C;
            a_iy0[i]     = oy * g.conv.stride_y - g.conv.pad_top;
            a_ix0[i]     = ox * g.conv.stride_x - g.conv.pad_left;
        }
        else
        {
            a_off[i] = (int64_t)gr * g.lda + col * 16;
            a_iy0[i] = a_ix0[i] = 0;
        }
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i)
    {
        const int c   = tid + i * NT;
        const int row = c / CPR, col = c % CPR;
        b_lds[i]      = BM * BK + row * BK + ((col ^ swz<CPR>(row)) << 4);
        b_off[i]      = (int64_t)row * g.Kp + col * 16;
    }

    v4i ra[A_CHUNKS], rb[B_CHUNKS];
    const bool gather = CONV && ((g.conv.C & 15) != 0 || ((uintptr_t)g.A & 15) != 0);

    auto load_tiles = [&](int k0)
    {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
        {
            const int k = k0 + a_col[i];
            v4i       v = {0, 0, 0, 0};
            if (k < g.K)
            {
                if (CONV && gather)
                {
                    // channel counts that are not a multiple of 16: a 16-byte piece crosses taps, every byte is looked up
                    uint32_t w[4] = {0, 0, 0, 0};
                    for (int b = 0; b < 16; ++b)
                    {
                        const int kb = k + b;
                        uint32_t  byte = 0;
                        if (kb < g.K)
                        {
                            const int tap = kb / g.conv.C;
                            const int c0  = kb - tap * g.conv.C;
                            const int ky  = tap / g.conv.KW;
                            const int kx  = tap - ky * g.conv.KW;
                            const int iy  = a_iy0[i] + ky * g.conv.dil_y;
                            const int ix  = a_ix0[i] + kx * g.conv.dil_x;
                            if (iy >= 0 && iy < g.conv.H && ix >= 0 && ix < g.conv.W)
                                byte = (uint8_t)A[a_off[i] + ((int64_t)iy * g.conv.W + ix) * g.conv.C + c0] ^ (FLIP_A ? 0x80u : 0u);
                            else
                                byte = g.conv.pad_word & 0xFFu;
                        }
                        w[b >> 2] |= byte << (8 * (b & 3));
                    }
                    v = (v4i){(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                }
                else if (CONV)
                {
                    const int tap = k / g.conv.C;
                    const int c0  = k - tap * g.conv.C;
                    const int ky  = tap / g.conv.KW;
                    const int kx  = tap - ky * g.conv.KW;
                    const int iy  = a_iy0[i] + ky * g.conv.dil_y;
                    const int ix  = a_ix0[i] + kx * g.conv.dil_x;
                    if (iy >= 0 && iy < g.conv.H && ix >= 0 && ix < g.conv.W)
                    {
                        v = *(const v4i *)(A + a_off[i] + ((int64_t)iy * g.conv.W + ix) * g.conv.C + c0);
                        if (FLIP_A)
                            v ^= (int)0x80808080;
                    }
                    else
                    {
                        const int pw = (int)g.conv.pad_word;
                        v            = (v4i){pw, pw, pw, pw};
                    }
                }
                else
                {
                    const int rem = g.K - k;
                    v = rem >= 16 ? *(const v4i *)(A + a_off[i] + k0) : load16_partial(A + a_off[i] + k0, rem);
                    if (FLIP_A)
                        v ^= (int)0x80808080;
                }
            }
            ra[i] = v;
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            rb[i] = *(const v4i *)(Bp + b_off[i] + k0);
    };
    auto store_tiles = [&](int stage)
    {
        char *s = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            *(v4i *)(s + a_lds[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i)
            *(v4i *)(s + b_lds[i]) = rb[i];
    };

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0;

    // operand read addresses: lane -> (row lane%32, 16-byte column lane/32) of a 32 x 32 operand block
    const int lr = lane & 31, lh = lane >> 5;
    int       a_rd[FM], b_rd[FN], a_sw[FM], b_sw[FN];
#pragma unroll
    for (int f = 0; f < FM; ++f)
    {
        const int row = wm * TM + f * 32 + lr;
        a_rd[f]       = row * BK;
        a_sw[f]       = swz<CPR>(row);
    }
#pragma unroll
    for (int f = 0; f < FN; ++f)
    {
        const int row = wn * TN + f * 32 + lr;
        b_rd[f]       = BM * BK + row * BK;
        b_sw[f]       = swz<CPR>(row);
    }

    const int nk = (g.K + BK - 1) / BK; // k tiles that hold real data (the packed B is zero beyond K)
    load_tiles(0);
    store_tiles(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt)
    {
        if (kt + 1 < nk)
            load_tiles((kt + 1) * BK);
        const char *s = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk)
        {
            v4i fa[FM], fb[FN];
#pragma unroll
            for (int f = 0; f < FM; ++f)
                fa[f] = *(const v4i *)(s + a_rd[f] + (((kk * 2 + lh) ^ a_sw[f]) << 4));
#pragma unroll
            for (int f = 0; f < FN; ++f)
                fb[f] = *(const v4i *)(s + b_rd[f] + (((kk * 2 + lh) ^ b_sw[f]) << 4));
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk)
            store_tiles((kt + 1) & 1);
        __syncthreads();
    }

    epilogue_store<EPI, FM, FN>(acc, g, m0 + wm * TM, n0 + wn * TN, lane, bz);
}

// ---- instantiation table -------------------------------------------------------------------------------------------
struct CfgEntry
{
    MfmaConfig cfg;
    int        threads;
    int        lds_bytes;
    const void *fn[3][2][2]; // [epi][flip][conv]
};

#define MI355_FN(BM, BN, BK, WM, WN, E, F, C) (const void *)gemm_mfma_kernel<BM, BN, BK, WM, WN, E, F, C>
#define MI355_CFG(NAME, BM, BN, BK, WM, WN)                                                                         \
    {                                                                                                               \
        {NAME, BM, BN, BK}, WM *WN * 64, 2 * (BM + BN) * BK,                                                         \
        {                                                                                                           \
            {{MI355_FN(BM, BN, BK, WM, WN, 0, false, false), nullptr},                                               \
             {MI355_FN(BM, BN, BK, WM, WN, 0, true, false), nullptr}},                                               \
                {{MI355_FN(BM, BN, BK, WM, WN, 1, false, false), MI355_FN(BM, BN, BK, WM, WN, 1, false, true)},      \
                 {MI355_FN(BM, BN, BK, WM, WN, 1, true, false), MI355_FN(BM, BN, BK, WM, WN, 1, true, true)}},       \
                {{MI355_FN(BM, BN, BK, WM, WN, 2, false, false), MI355_FN(BM, BN, BK, WM, WN, 2, false, true)},      \
                 {MI355_FN(BM, BN, BK, WM, WN, 2, true, false), MI355_FN(BM, BN, BK, WM, WN, 2, true, true)}},       \
        }                                                                                                           \
    }

static const CfgEntry g_cfgs[] = {
    MI355_CFG("mfma_256x128x64", 256, 128, 64, 2, 2),
    MI355_CFG("mfma_128x128x64", 128, 128, 64, 2, 2),
    MI355_CFG("mfma_128x64x64", 128, 64, 64, 2, 2),
    MI355_CFG("mfma_64x64x64", 64, 64, 64, 2, 2),
};

int mfma_num_configs()
{
    return (int)(sizeof(g_cfgs) / sizeof(g_cfgs[0]));
}
MfmaConfig mfma_config(int idx)
{
    return g_cfgs[idx].cfg;
}

int mfma_launch(int cfg_idx, int epi, bool flip_a, bool conv, const GemmArgs &args, int batch, hipStream_t s)
{
    if (cfg_idx < 0 || cfg_idx >= mfma_num_configs() || epi < 0 || epi > 2)
        return (int)hipErrorInvalidValue;
    const CfgEntry &c  = g_cfgs[cfg_idx];
    const void     *fn = c.fn[epi][flip_a ? 1 : 0][conv ? 1 : 0];
    if (fn == nullptr)
        return (int)hipErrorInvalidValue;
    // shapes the kernel assumes: loop bound a multiple of BK inside the packed panel, tiles cover the output
    if (args.Kp % c.cfg.BK != 0 || args.K > args.Kp || args.tiles_m * c.cfg.BM < args.M ||
        args.tiles_n * c.cfg.BN < args.N || args.tiles_n * c.cfg.BN > round_up(args.N, PACK_N_ALIGN) || args.M < 1)
        return (int)hipErrorInvalidValue;
    if (c.lds_bytes > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, c.lds_bytes);
        if (e != hipSuccess)
            return (int)e;
    }
    GemmArgs a      = args;
    void    *kargs[] = {&a};
    dim3     grid(args.tiles_m * args.tiles_n, 1, batch), block(c.threads);
    return (int)hipLaunchKernel(fn, grid, block, kargs, c.lds_bytes, s);
}
} // namespace mi355
