// K3: bandwidth-bound GEMM for M <= 64 (decode-shaped: one token batch against a large weight matrix).
//
// The reference has no dedicated kernel above M == 1 (GemvPretransposed, src/core/NEON/kernels/arm_gemm/gemm_qint8.cpp:75-79)
// and otherwise runs its hybrid kernels; here the whole run is one streaming pass over B at HBM speed.
//
// B is packed at prepare time into 1 KiB blocks of 16 columns x 64 k in matrix-core operand order
// (Bs[Np/16][Kp/64][64 lanes][16 bytes]), so every wave-wide load is one contiguous, fully coalesced 1 KiB read and a
// column group's K range is one contiguous stream. A block owns NG groups of 16 output columns; its WAVES waves split
// the k blocks, each keeping UNROLL steps of loads in flight, multiply with v_mfma_i32_16x16x64_i8 (MR blocks of 16 A
// rows, padded with zeros; A itself is tiny and stays in L2), reduce the partial 16 x 16 accumulators through LDS, and
// wave r applies the fused offset / requantisation epilogue to row block r. The kernel lives on memory-level parallelism: every block of the grid
// should be resident at once, so the register footprint is kept small (the K tail has its own one-step loop) and the
// number of waves per block is chosen from the number of column groups.
#include "internal.hpp"

#include <atomic>
#include <cstdlib>

namespace mi355
{
typedef int v4i __attribute__((ext_vector_type(4)));


// STAGE_A: a wave's K slice of A is at most 4 KiB / WAVES per row (K <= 4096); the row pitch of its staged copy adds
// 64 bytes, which spreads the 8 rows an operand read touches over the LDS banks
constexpr int sk_a_slice(int waves) { return 4096 / waves; }
constexpr int sk_a_pitch(int waves) { return sk_a_slice(waves) + 64; }
template <int EPI, bool FLIP_A, int NG, int SK_WAVES, int SK_UNROLL, bool STAGE_A, int MR, bool STEP_A = false,
          int STEP_KB = (MR == 4 ? 4 : 8)>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(GemmArgs g)
{
    static_assert(MR >= 1 && MR <= SK_WAVES && (!STAGE_A || MR == 1), "row blocks");
    static_assert(!STEP_A || (!STAGE_A && SK_UNROLL == 8), "per-step staging: steps of 8 k blocks");
    __shared__ __attribute__((aligned(16))) int32_t red[SK_WAVES][NG][64][4];
    extern __shared__ __attribute__((aligned(16))) char a_stage[]; // STAGE_A: [SK_WAVES][M <= 8][sk_a_pitch(SK_WAVES)]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int ng0  = blockIdx.x * NG; // first of this block's NG groups of 16 columns
    const int KB   = (int)(g.Kp / 64);
    const int NGT  = (int)((g.N + 15) / 16);

    // waves 0..MR-1 apply the epilogue to column ng0*16 + (lane%16) + 16*n: fetch its per-column constants now, so
    // that their latency is hidden behind the B stream instead of following it
    const EpiParams &p = g.epi;
    int32_t          cv[NG], mu[NG], sh[NG];
    float            bf[NG];
#pragma unroll
    for (int n = 0; n < NG; ++n)
    {
        const int j = min((ng0 + n) * 16 + (lane & 15), g.N - 1);
        cv[n] = 0, mu[n] = p.mult_s, sh[n] = p.shift_s, bf[n] = 0.f;
        if (wave < MR)
        {
            cv[n] = p.colvec[j];
            if (EPI == EPI_FIXEDPOINT && p.mult)
            {
                mu[n] = p.mult[j];
                sh[n] = p.shift[j];
            }
            if (EPI == EPI_F32 && p.bias_f32)
                bf[n] = p.bias_f32[j];
        }
    }

    // this wave's contiguous range of k blocks
    const int per  = (KB + SK_WAVES - 1) / SK_WAVES;
    const int kb0  = wave * per;
    const int kb1  = min(KB, kb0 + per);

    const int   arow   = lane & 15;
    const int   akc    = (lane >> 4) * 16;
    bool          a_live[MR];
    const int8_t *a_ptr[MR]; // rows past M re-read row M-1 and multiply as zeros
#pragma unroll
    for (int rb = 0; rb < MR; ++rb)
    {
        a_live[rb] = rb * 16 + arow < g.M;
        a_ptr[rb]  = g.A + (int64_t)min(rb * 16 + arow, g.M - 1) * g.lda + akc;
    }
    const int8_t *b_ptr[NG];
#pragma unroll
    for (int n = 0; n < NG; ++n)
        b_ptr[n] = g.Bp + ((int64_t)min(ng0 + n, NGT - 1) * KB * 64 + lane) * 16;

    v4i acc[MR][NG];
#pragma unroll
    for (int rb = 0; rb < MR; ++rb)
#pragma unroll
        for (int n = 0; n < NG; ++n)
            acc[rb][n] = (v4i){0, 0, 0, 0};
    const v4i zero4 = {0, 0, 0, 0};
    int       kb    = kb0;

    // STAGE_A (M <= 8, every wave's K slice at most A_SLICE bytes per row, K a multiple of 64, 16-byte aligned rows): the wave
    // copies its slice of A into LDS once, with all 64 lanes per load, and takes the operand blocks from there.
    // Loading them from global memory inside the stream costs one half-empty load instruction (rows 8..15 are padding)
    // per B load and 16 % of the kernel's time, although A never leaves the L2.
    constexpr int A_SLICE = sk_a_slice(SK_WAVES), A_PITCH = sk_a_pitch(SK_WAVES);
    constexpr int NA      = 8 * A_SLICE / 1024; // load instructions (1 KiB each) that cover 8 rows of a slice
    constexpr int LPR     = A_SLICE / 16;       // lanes per row
    char *a_lds = a_stage + (STEP_A ? wave * MR * 16 * (STEP_KB * 64 + 16) : wave * 8 * A_PITCH);
    v4i   ta[STAGE_A ? NA : 1];
    const int a_sr = lane / LPR, a_sc = (lane % LPR) * 16; // this lane's row (of 1024 / A_SLICE per load) and column
    if (STAGE_A)
    {
        // branch-free (a branch per row would put a full wait behind every load): rows past M re-read row M-1 into
        // staging rows nobody reads, lanes past the slice re-read its first 16 bytes into columns nobody reads
        const int slice = max(kb1 - kb0, 0) * 64; // bytes per row, <= A_SLICE
        const int col   = a_sc < slice ? a_sc : 0;
        const int8_t *src = g.A + (int64_t)min(kb0, KB - 1) * 64 + col;
#pragma unroll
        for (int i = 0; i < NA; ++i)
            ta[i] = *(const v4i *)(src + (int64_t)min(i * (1024 / A_SLICE) + a_sr, g.M - 1) * g.lda);
    }
    const char *a_frag = a_lds + arow * A_PITCH + akc; // this lane's piece of the operand block of k block kb0
    // whole steps inside the wave's range and inside K: straight-line loads, all in flight together; the loads of the
    // next step directly follow the matrix instructions of this one.
    v4i  fb[SK_UNROLL][NG];
    auto whole_step = [&](int k) { return k + SK_UNROLL <= kb1 && (k + SK_UNROLL) * 64 <= g.K; };
    auto load_b     = [&](int k)
    {
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
            for (int n = 0; n < NG; ++n)
                fb[u][n] = __builtin_nontemporal_load((const v4i *)(b_ptr[n] + (int64_t)(k + u) * 1024));
    };
    // STAGE_A: the first step of the B stream is issued before the wave waits for its slice of A. Loads return in order,
    // so the wait for A (the older loads) does not wait for B, and one memory latency leaves the critical path
    // (M = 8, N = 11008, K = 4096: 9.7 -> 9.4 us).
    bool more = false;
    if (STAGE_A)
    {
        more = whole_step(kb);
        if (more)
            load_b(kb);
#pragma unroll
        for (int i = 0; i < NA; ++i)
        {
            if (FLIP_A)
                ta[i] ^= (int)0x80808080;
            *(v4i *)(a_lds + (i * (1024 / A_SLICE) + a_sr) * A_PITCH + a_sc) = ta[i];
        }
    }
    if constexpr (STEP_A)
    {
        // More than 8 rows: the bytes of A that a step needs go through LDS, STEP_KB k blocks at a time - loads of 2
        // (or 4) rows x 512 (256) contiguous bytes, whole cache lines with every lane busy, instead of gathers of 16
        // rows x 64 bytes, which cost the L2 twice the requests. No branches (a branch per load would put a full wait
        // behind every load): rows past M re-read row M-1 and are multiplied into accumulator rows that are never stored. LDS operations of one wave execute in order, so
        // the next pass's writes cannot overtake this pass's reads.
        constexpr int SKB   = STEP_KB;              // k blocks per staging pass
        constexpr int LPR   = SKB * 4;               // lanes per row (16 bytes each)
        constexpr int RPL   = 64 / LPR;              // rows per load instruction
        constexpr int PITCH = SKB * 64 + 16;         // 16 rows of an operand read fall into 16 different bank groups
        const int     sub = lane / LPR, col = (lane % LPR) * 16;
        more = whole_step(kb);
        if (more)
            load_b(kb);
        while (more)
        {
#pragma unroll
            for (int h = 0; h < SK_UNROLL / SKB; ++h)
            {
#pragma unroll
                for (int c = 0; c < MR; ++c)
                {
                    v4i ts[16 / RPL];
#pragma unroll
                    for (int q = 0; q < 16 / RPL; ++q)
                        ts[q] = *(const v4i *)(g.A + (int64_t)min(c * 16 + q * RPL + sub, g.M - 1) * g.lda +
                                               (int64_t)(kb + h * SKB) * 64 + col);
#pragma unroll
                    for (int q = 0; q < 16 / RPL; ++q)
                    {
                        if (FLIP_A)
                            ts[q] ^= (int)0x80808080;
                        *(v4i *)(a_lds + (c * 16 + q * RPL + sub) * PITCH + col) = ts[q];
                    }
                }
#pragma unroll
                for (int u = h * SKB; u < (h + 1) * SKB; ++u)
                {
                    v4i fa[MR];
#pragma unroll
                    for (int rb = 0; rb < MR; ++rb)
                        fa[rb] = *(const v4i *)(a_lds + (rb * 16 + arow) * PITCH + (u - h * SKB) * 64 + akc);
#pragma unroll
                    for (int rb = 0; rb < MR; ++rb)
#pragma unroll
                        for (int n = 0; n < NG; ++n)
                            acc[rb][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[rb], fb[u][n], acc[rb][n], 0, 0, 0);
                }
            }
            kb += SK_UNROLL;
            more = whole_step(kb);
            if (more)
                load_b(kb);
        }
    }
    else if constexpr (MR == 1)
    {
        if (!STAGE_A)
        {
            more = whole_step(kb);
            if (more)
                load_b(kb);
        }
        while (more)
        {
            // staged operands are read in two halves (the scheduler would otherwise hoist all reads and hold 8
            // operand blocks next to the 8 blocks of B: 86 registers, one too few waves per SIMD for the 8-wave variant)
            constexpr int HALVES = STAGE_A ? 2 : 1, HU = SK_UNROLL / HALVES;
#pragma unroll
            for (int h = 0; h < HALVES; ++h)
            {
                v4i fa[HU];
#pragma unroll
                for (int u = 0; u < HU; ++u)
                    fa[u] = zero4;
                if (a_live[0])
                {
#pragma unroll
                    for (int u = 0; u < HU; ++u)
                    {
                        if (STAGE_A)
                            fa[u] = *(const v4i *)(a_frag + (kb + h * HU + u - kb0) * 64);
                        else
                        {
                            fa[u] = *(const v4i *)(a_ptr[0] + (int64_t)(kb + u) * 64);
                            if (FLIP_A)
                                fa[u] ^= (int)0x80808080;
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < HU; ++u)
#pragma unroll
                    for (int n = 0; n < NG; ++n)
                        acc[0][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[u], fb[h * HU + u][n], acc[0][n], 0, 0, 0);
                if (HALVES > 1)
                    __builtin_amdgcn_sched_barrier(0);
            }
            kb += SK_UNROLL;
            more = whole_step(kb);
            if (more)
                load_b(kb);
        }
    }
    else
    {
        // Several row blocks: the operand blocks of A come from the L2 with every step, so a wave would wait a full
        // memory latency per step. Two register sets instead: the loads of step s+1 (B and A, branch-free - rows past
        // M re-read row M-1 and are zeroed afterwards) are issued before the matrix instructions of step s.
        v4i  fa[SK_UNROLL][MR], fb2[SK_UNROLL][NG], fa2[SK_UNROLL][MR];
        auto load_ab = [&](v4i(&b)[SK_UNROLL][NG], v4i(&a)[SK_UNROLL][MR], int k)
        {
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u)
            {
#pragma unroll
                for (int n = 0; n < NG; ++n)
                    b[u][n] = __builtin_nontemporal_load((const v4i *)(b_ptr[n] + (int64_t)(k + u) * 1024));
#pragma unroll
                for (int rb = 0; rb < MR; ++rb)
                    a[u][rb] = *(const v4i *)(a_ptr[rb] + (int64_t)(k + u) * 64);
            }
        };
        auto multiply = [&](v4i(&b)[SK_UNROLL][NG], v4i(&a)[SK_UNROLL][MR])
        {
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
                for (int rb = 0; rb < MR; ++rb)
                {
                    if (FLIP_A)
                        a[u][rb] ^= (int)0x80808080;
                    if (!a_live[rb])
                        a[u][rb] = zero4;
#pragma unroll
                    for (int n = 0; n < NG; ++n)
                        acc[rb][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[u][rb], b[u][n], acc[rb][n], 0, 0, 0);
                }
        };
        more = whole_step(kb);
        if (more)
            load_ab(fb, fa, kb);
        while (more)
        {
            const bool more2 = whole_step(kb + SK_UNROLL);
            if (more2)
                load_ab(fb2, fa2, kb + SK_UNROLL);
            multiply(fb, fa);
            kb += SK_UNROLL;
            if (!more2)
                break;
            more = whole_step(kb + SK_UNROLL);
            if (more)
                load_ab(fb, fa, kb + SK_UNROLL);
            multiply(fb2, fa2);
            kb += SK_UNROLL;
        }
    }
    // remaining k blocks one at a time, with the guarded loads of the K tail
    for (; kb < kb1; ++kb)
    {
        v4i fa[MR], fb[NG];
#pragma unroll
        for (int n = 0; n < NG; ++n)
            fb[n] = *(const v4i *)(b_ptr[n] + (int64_t)kb * 1024);
        const int rem = g.K - (kb * 64 + akc);
#pragma unroll
        for (int rb = 0; rb < MR; ++rb)
        {
            fa[rb] = zero4;
            if (STAGE_A)
            {
                if (a_live[rb])
                    fa[rb] = *(const v4i *)(a_frag + (kb - kb0) * 64);
            }
            else if (a_live[rb] && rem > 0)
            {
                fa[rb] = rem >= 16 ? *(const v4i *)(a_ptr[rb] + (int64_t)kb * 64)
                                   : load16_partial(a_ptr[rb] + (int64_t)kb * 64, rem);
                if (FLIP_A)
                    fa[rb] ^= (int)0x80808080;
            }
        }
#pragma unroll
        for (int rb = 0; rb < MR; ++rb)
#pragma unroll
            for (int n = 0; n < NG; ++n)
                acc[rb][n] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[rb], fb[n], acc[rb][n], 0, 0, 0);
    }

    // one row block at a time through the same LDS: wave rb sums and finishes row block rb
    v4i sum[NG];
#pragma unroll
    for (int n = 0; n < NG; ++n)
        sum[n] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int rb = 0; rb < MR; ++rb)
    {
        if (rb > 0)
            __syncthreads();
#pragma unroll
        for (int n = 0; n < NG; ++n)
            *(v4i *)&red[wave][n][lane][0] = acc[rb][n];
        __syncthreads();
        if (wave == rb)
        {
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w)
#pragma unroll
                for (int n = 0; n < NG; ++n)
                    sum[n] += *(const v4i *)&red[w][n][lane][0];
        }
    }
    if (wave >= MR)
        return;

    // accumulator r of lane l is row 16*rb + 4*(l/16) + r, column l%16
#pragma unroll
    for (int n = 0; n < NG; ++n)
    {
        const int j = (ng0 + n) * 16 + (lane & 15);
        if (j >= g.N)
            continue;
#pragma unroll
        for (int r = 0; r < 4; ++r)
        {
            const int i = 16 * wave + 4 * (lane >> 4) + r;
            if (i < g.M)
            {
                const int32_t rv  = p.rowvec ? p.rowvec[i] : 0;
                const int64_t idx = (int64_t)i * g.ldd + j;
                if (EPI == EPI_S32)
                    ((int32_t *)g.D)[idx] = (int32_t)((uint32_t)sum[n][r] + (uint32_t)cv[n] + (uint32_t)rv +
                                                      (p.accumulate ? (uint32_t)((int32_t *)g.D)[idx] : 0u));
                else if (EPI == EPI_FIXEDPOINT)
                    ((int8_t *)g.D)[idx] = (int8_t)epi_fixedpoint(sum[n][r], cv[n], rv, mu[n], sh[n], p);
                else
                    ((float *)g.D)[idx] = epi_f32(sum[n][r], (int32_t)((uint32_t)cv[n] + (uint32_t)rv), bf[n],
                                                  p.bias_f32 != nullptr, p, p.accumulate ? ((float *)g.D)[idx] : 0.f);
            }
        }
    }
}

// A kernel that needs more than 48 KiB of dynamic LDS has to be told so once per device
static int raise_lds_limit(const void *fn, size_t lds, std::atomic<uint32_t> &done)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32)
        return (int)hipErrorInvalidDevice;
    if (done.load(std::memory_order_acquire) & (1u << dev))
        return 0;
    const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e == hipSuccess)
        done.fetch_or(1u << dev, std::memory_order_release);
    return (int)e;
}

template <int NG, int WAVES, int UNROLL, bool STAGE_A, int MR = 1, bool STEP_A = false>
static int skinny_launch_v(int epi, bool flip_a, const GemmArgs &a, hipStream_t s)
{
    const int    groups = (a.N + 15) / 16;
    const dim3   grid((groups + NG - 1) / NG), block(WAVES * 64);
    const size_t lds = STAGE_A ? (size_t)WAVES * 8 * sk_a_pitch(WAVES) : (STEP_A ? (size_t)WAVES * MR * 16 * ((MR == 4 ? 4 : 8) * 64 + 16) : 0);
    if (epi != EPI_S32 && epi != EPI_FIXEDPOINT && epi != EPI_F32)
        return (int)hipErrorInvalidValue;
    static const void *const fns[3][2] = {
        {(const void *)gemm_skinny_kernel<EPI_S32, false, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>,
         (const void *)gemm_skinny_kernel<EPI_S32, true, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>},
        {(const void *)gemm_skinny_kernel<EPI_FIXEDPOINT, false, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>,
         (const void *)gemm_skinny_kernel<EPI_FIXEDPOINT, true, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>},
        {(const void *)gemm_skinny_kernel<EPI_F32, false, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>,
         (const void *)gemm_skinny_kernel<EPI_F32, true, NG, WAVES, UNROLL, STAGE_A, MR, STEP_A>}};
    static std::atomic<uint32_t> lds_raised[3][2];
    const void *fn = fns[epi][flip_a ? 1 : 0];
    if (lds > 48 * 1024)
    {
        const int e = raise_lds_limit(fn, lds, lds_raised[epi][flip_a ? 1 : 0]);
        if (e)
            return e;
    }
    GemmArgs copy    = a;
    void    *kargs[] = {&copy};
    return (int)hipLaunchKernel(fn, grid, block, kargs, lds, s);
}

// Environment overrides for experiments, read once: MI355_SKINNY_WAVES (4 or 8; anything else is ignored),
// MI355_SKINNY_NG (column groups per workgroup), MI355_SKINNY_NO_STAGE (A operands straight from global memory)
struct SkinnyEnv
{
    int  waves = 0, ng = 0;
    bool no_stage = false;
    SkinnyEnv()
    {
        const char *w = getenv("MI355_SKINNY_WAVES"), *n = getenv("MI355_SKINNY_NG");
        if (w && (atoi(w) == 4 || atoi(w) == 8))
            waves = atoi(w);
        if (n && atoi(n) >= 1 && atoi(n) <= 4)
            ng = atoi(n);
        no_stage = getenv("MI355_SKINNY_NO_STAGE") != nullptr;
    }
};

int skinny_launch(int epi, bool flip_a, const GemmArgs &args, hipStream_t s)
{
    if (args.M < 1 || args.M > SKINNY_MAX_M || args.Kp % 64 != 0 || args.K > args.Kp)
        return (int)hipErrorInvalidValue;
    static const SkinnyEnv env;
    const int groups = (args.N + 15) / 16;
    const int KB     = (int)(args.Kp / 64);
    // Up to 8 rows every wave copies its K slice of A (at most 1 KiB per row) into LDS once and takes its operands
    // from there; that needs nothing to guard
    const bool stage_ok = args.M <= 8 && args.K == args.Kp && args.K % 64 == 0 && args.lda % 16 == 0 &&
                          ((uintptr_t)args.A & 15) == 0 && !env.no_stage;
    // The kernel lives on loads in flight: 8 waves per workgroup while each of them still has at least one whole
    // step of 8 k blocks and all workgroups are resident together (24 waves of this size per compute unit), 4 otherwise
    int waves = (groups >= 512 && !(stage_ok && KB >= 64 && (int64_t)groups * 8 <= 24 * 256)) ? 4 : 8;
    if (env.waves)
        waves = env.waves;
    const int  per   = (KB + waves - 1) / waves;
    const bool stage = stage_ok && per * 64 <= sk_a_slice(waves);
    // more than 8 rows: per-step staging (dword-aligned rows are enough: the staging loads are plain 16-byte loads)
    const bool step = args.M > 8 && args.lda % 4 == 0 && ((uintptr_t)args.A & 3) == 0 && !env.no_stage;
    // (17..24 rows: the gathers of the unstaged variants below re-read row M-1 for the missing rows of the second
    // block, which costs less than staging 32 rows)
    if (args.M > 24 && step)
    {
        // LDS: 8.25 KiB per wave and block of 16 rows; a workgroup covers 2 column groups when there are many
        const int ng     = env.ng ? (env.ng >= 2 ? 2 : 1) : (groups >= 512 ? 2 : 1);
        const int blocks = (groups + ng - 1) / ng;
        if (args.M > 32)
            return ng == 2 ? skinny_launch_v<2, 4, 8, false, 4, true>(epi, flip_a, args, s)
                           : skinny_launch_v<1, 4, 8, false, 4, true>(epi, flip_a, args, s);
        const int w = env.waves ? env.waves : (blocks >= 320 ? 4 : 8);
        if (ng == 2)
            return w == 4 ? skinny_launch_v<2, 4, 8, false, 2, true>(epi, flip_a, args, s)
                          : skinny_launch_v<2, 8, 8, false, 2, true>(epi, flip_a, args, s);
        return w == 4 ? skinny_launch_v<1, 4, 8, false, 2, true>(epi, flip_a, args, s)
                      : skinny_launch_v<1, 8, 8, false, 2, true>(epi, flip_a, args, s);
    }
    if (args.M > 16)
    {
        // More than one block of 16 rows: A (L2 resident) is re-read once per block of the grid, which costs as much as
        // the B stream unless a block covers several column groups - as many as still leave a few hundred blocks.
        const int mr = args.M > 32 ? 4 : 2;
        int       ng = groups >= 1024 ? 4 : (groups >= 512 ? 2 : 1);
        if (env.ng)
            ng = env.ng;
        ng = ng >= 4 && mr == 4 ? 4 : (ng >= 2 ? 2 : 1);
        const int blocks = (groups + ng - 1) / ng;
        const int w      = env.waves ? env.waves : (blocks >= 320 ? 4 : 8);
#define MI355_SKV(NG_, MR_)                                                                          \
    (w == 4 ? skinny_launch_v<NG_, 4, 2, false, MR_>(epi, flip_a, args, s)                           \
            : skinny_launch_v<NG_, 8, 2, false, MR_>(epi, flip_a, args, s))
        if (mr == 2)
            return ng == 2 ? MI355_SKV(2, 2) : MI355_SKV(1, 2);
        return ng == 4 ? MI355_SKV(4, 4) : (ng == 2 ? MI355_SKV(2, 4) : MI355_SKV(1, 4));
#undef MI355_SKV
    }
    // the waves of the unstaged / per-step variants follow the old rule
    const int w1 = env.waves ? env.waves : (groups >= 512 ? 4 : 8);
    if (step) // 9..16 rows
        return w1 == 4 ? skinny_launch_v<1, 4, 8, false, 1, true>(epi, flip_a, args, s)
                       : skinny_launch_v<1, 8, 8, false, 1, true>(epi, flip_a, args, s);
    if (stage)
        return waves == 4 ? skinny_launch_v<1, 4, 8, true>(epi, flip_a, args, s) : skinny_launch_v<1, 8, 8, true>(epi, flip_a, args, s);
    return w1 == 4 ? skinny_launch_v<1, 4, 8, false>(epi, flip_a, args, s) : skinny_launch_v<1, 8, 8, false>(epi, flip_a, args, s);
}
} // namespace mi355
