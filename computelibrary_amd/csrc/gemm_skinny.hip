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

#include <algorithm>
#include <atomic>
#include <type_traits>
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

    // entry blockIdx.y of a batch: every operand moves on by its batch stride (one launch covers the batch)
    if (gridDim.y > 1)
    {
        const int64_t bz = blockIdx.y;
        g.A += bz * g.a_batch_stride;
        g.Bp += bz * g.bp_batch_stride;
        g.D = (char *)g.D + bz * g.d_batch_stride * (EPI == EPI_FIXEDPOINT ? 1 : 4);
        g.epi.colvec += bz * g.epi.colvec_batch_stride;
        if (g.epi.rowvec)
            g.epi.rowvec += bz * g.epi.rowvec_batch_stride;
    }
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


// M <= 8, K <= 4096: the stage-once form. One workgroup of 16 waves per compute unit walks the column groups
// blockIdx.x, blockIdx.x + gridDim.x, ... (at most ONCE_MAX_GROUPS of them); wave w owns the k blocks
// [w * PER, (w + 1) * PER) of every group and copies its slice of A into LDS once for all groups. With one workgroup per
// group, A (which never leaves the L2) crosses the compute unit's vector-memory path once per group and takes a third
// of its requests; here it crosses once per compute unit. One group of B loads is in flight per wave, refilled half by half (see ONE_SLOT). Partial sums
// meet in double-buffered LDS (one barrier per group) and 8 x 16 threads finish one output each, so the only work
// behind the last byte of B is one short chain; their per-column constants are fetched before the stream starts.
constexpr int ONCE_WAVES      = 16;
constexpr int ONCE_MAX_GROUPS = 4;
// The arguments this kernel uses, packed into 136 bytes: it reads all of them in one batch of scalar loads before
// anything else. With the general argument block (three times the size, the used fields scattered over it) the
// compiler fetched some fields where they were first used, which put a second round trip to memory in front of the B
// stream and a third one behind it, in the epilogue; the number of workgroups is passed for the same reason (gridDim is
// a hidden argument behind the block).
struct OnceArgs
{
    const int8_t  *A, *Bp;
    void          *D;
    const int32_t *colvec, *rowvec, *mult, *shift;
    const float   *bias_f32;
    int64_t        lda, ldd;
    int32_t        M, N, KB, grid;
    int32_t        result_offset, stage, lo, hi;
    float          scale, act_min, act_max;
    int32_t        has_offsets, accumulate, act_twice;
};
// One output of the stage-once kernels: the reduced sum, its column term c, multiplier (or float bias bits) m, shift sh
// and row term rv through epilogue EPI into element idx of D
#define MI355_GLOBAL __attribute__((address_space(1)))
template <int EPI>
__device__ __forceinline__ void once_store_output(MI355_GLOBAL char *gD, int64_t idx, int32_t sum, int32_t c, int32_t m, int32_t sh,
                                                  int32_t rv, bool has_bias, const EpiParams &p)
{
    if (EPI == EPI_S32)
        ((MI355_GLOBAL int32_t *)gD)[idx] =
            (int32_t)((uint32_t)sum + (uint32_t)c + (uint32_t)rv + (p.accumulate ? (uint32_t)((MI355_GLOBAL int32_t *)gD)[idx] : 0u));
    else if (EPI == EPI_FIXEDPOINT)
    {
        const int32_t v = (int32_t)((uint32_t)sum + (uint32_t)c + (uint32_t)rv);
        int32_t       q;
        if (p.stage == 0 && m >= 0 && sh > -32 && sh < 32)
            // the branch-free form of the same arithmetic (see fast_requant), its constants derived here
            q = fast_requant(v, (int32_t)((uint32_t)m << 1), (uint32_t)m >= 0x40000000u ? -1 : 0, sh < 0 ? -sh : 0, sh > 1 ? sh - 1 : 0,
                             sh > 0 ? 1 : 0, p.result_offset, p.lo, p.hi);
        else
            q = epi_fixedpoint(sum, c, rv, m, sh, p);
        ((MI355_GLOBAL int8_t *)gD)[idx] = (int8_t)q;
    }
    else
        ((MI355_GLOBAL float *)gD)[idx] = epi_f32(sum, (int32_t)((uint32_t)c + (uint32_t)rv), __int_as_float(m), has_bias, p,
                                                  p.accumulate ? ((MI355_GLOBAL float *)gD)[idx] : 0.f);
}
#undef MI355_GLOBAL

// bytes from one staged row of A to the next: 8 / 16 rows keep the pitch they were tuned with; 32 rows take the smallest
// pitch that still spreads the rows over the banks (an odd number of 16-byte pieces), or the slices would not fit
__host__ __device__ constexpr int once_pitch(int rows, int per)
{
    return per * 64 + (rows > 16 ? 16 : 64);
}

// ROWS: rows of A - 8 (half of the matrix instruction's rows are padding), 16, 32 (two blocks of 16 rows: two matrix
// instructions per B operand block) or 64 (four blocks). Up to 32 rows a workgroup has 16 waves and every wave stages
// its K slice of A in LDS; 64 rows x 4096 bytes would not fit there, and need not: the operand blocks of A stay in
// registers for the whole kernel, so with 64 rows a workgroup has 8 waves (256 registers each: 128 of them hold A) and
// gathers the blocks straight from global memory, once.
template <int EPI, bool FLIP_A, int PER, bool MULTI, int ROWS, int WAVES = ONCE_WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_once_kernel(OnceArgs g)
{
    static_assert(ROWS == 8 || ROWS == 16 || ROWS == 32 || ROWS == 64, "rows");
    static_assert((ROWS == 64) == (WAVES == 8) && (WAVES == 8 || WAVES == ONCE_WAVES), "waves");
    constexpr bool A_GLOBAL = ROWS == 64;      // operand blocks of A straight from global memory
    constexpr int RB    = ROWS / 16 > 0 ? ROWS / 16 : 1; // blocks of 16 rows
    constexpr int RL    = ROWS == 8 ? 32 : 64; // lanes of a wave that hold results (per block of rows)
    constexpr int SLICE = PER * 64, PITCH = once_pitch(ROWS, PER); // bytes of a row of A per wave
    constexpr int NA    = ROWS * SLICE / 1024 > 0 ? ROWS * SLICE / 1024 : 1; // 1 KiB loads that cover the rows of a slice
    constexpr int LPR   = SLICE / 16;                                        // lanes per row
    constexpr int RPL   = 64 / LPR > ROWS ? ROWS : 64 / LPR;                 // rows per load
    // partial results [2][wave][block of rows][lane][4]: for 32 rows they take over the staging area once every wave
    // has its operands of A in registers (the two together would not fit)
    constexpr bool RED_IN_STAGE = RB > 1 || (ROWS == 16 && PER == 8); // (16 rows of 8 k blocks per wave fill LDS as well)
    __shared__ __attribute__((aligned(16))) int32_t red_own[RED_IN_STAGE ? 1 : 2 * WAVES * RB * RL * 4];
    __shared__ int32_t                              par[4][64]; // [vector][group * 16 + column]; row vector: [3][row]
    extern __shared__ __attribute__((aligned(16))) char a_stage[]; // [WAVES][ROWS][PITCH] (nothing staged with 64 rows)
    // (the launch sizes the dynamic area for the larger of the two)
    int32_t *const red = RED_IN_STAGE ? (int32_t *)a_stage : red_own;
    // red[((buf * WAVES + wave) * RB + rb) * RL + lane][4]

    // Everything is pinned in registers here, so that it is all fetched before this point. A pointer that went through the
    // asm as an integer is a generic pointer no more: it comes back as a pointer to global memory (generic loads would
    // wait for LDS and memory alike).
#define MI355_GLOBAL __attribute__((address_space(1)))
    uintptr_t u_a = (uintptr_t)g.A, u_b = (uintptr_t)g.Bp, u_d = (uintptr_t)g.D, u_cv = (uintptr_t)g.colvec, u_rv = (uintptr_t)g.rowvec,
              u_mu = (uintptr_t)g.mult, u_sh = (uintptr_t)g.shift, u_bf = (uintptr_t)g.bias_f32;
    asm volatile(""
                 : "+s"(g.result_offset), "+s"(g.stage), "+s"(g.lo), "+s"(g.hi), "+s"(g.scale), "+s"(g.act_min), "+s"(g.act_max),
                   "+s"(g.has_offsets), "+s"(g.accumulate), "+s"(g.act_twice), "+s"(g.lda), "+s"(g.ldd), "+s"(g.M), "+s"(g.N),
                   "+s"(g.KB), "+s"(g.grid), "+s"(u_a), "+s"(u_b), "+s"(u_d), "+s"(u_cv), "+s"(u_rv), "+s"(u_mu), "+s"(u_sh),
                   "+s"(u_bf));
    const MI355_GLOBAL int8_t *const  gA = (const MI355_GLOBAL int8_t *)u_a, *const gB = (const MI355_GLOBAL int8_t *)u_b;
    MI355_GLOBAL char *const          gD = (MI355_GLOBAL char *)u_d;
    const MI355_GLOBAL int32_t *const g_colvec = (const MI355_GLOBAL int32_t *)u_cv, *const g_rowvec = (const MI355_GLOBAL int32_t *)u_rv,
                                     *const g_mult = (const MI355_GLOBAL int32_t *)u_mu, *const g_shift = (const MI355_GLOBAL int32_t *)u_sh,
                                     *const g_bias = (const MI355_GLOBAL int32_t *)u_bf;
    const bool has_bias = u_bf != 0;
    EpiParams  p{};
    p.result_offset = g.result_offset, p.stage = g.stage, p.lo = g.lo, p.hi = g.hi;
    p.scale = g.scale, p.act_min = g.act_min, p.act_max = g.act_max;
    p.has_offsets = g.has_offsets, p.accumulate = g.accumulate, p.act_twice = g.act_twice;

    const int lane = threadIdx.x & 63;
    // (8 k blocks per wave: the wave index as a scalar, so that the addresses of the B blocks are a scalar base plus one
    // per-lane offset - as per-lane 64-bit addresses, all computed ahead, they pushed the B blocks out of the registers)
    const int wave = (PER == 8 && ROWS < 64) ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : (int)(threadIdx.x >> 6);
    const int KB   = g.KB;
    const int NGT  = (g.N + 15) / 16;
    const int G    = g.grid; // == gridDim.x
    const int mine = (NGT - (int)blockIdx.x + G - 1) / G; // column groups of this workgroup, 1..ONCE_MAX_GROUPS
    const int kb0  = wave * PER;
    const bool busy = kb0 < KB; // K < 1024 * PER leaves the last waves without k blocks

    // The epilogue's constants: 4 vectors (column term, multiplier or float bias, shift, row term) x 4 groups x 16 columns
    // are one dword per lane of four waves. Wave w fetches vector w % 4, before anything else - every wave, without a
    // condition (behind a branch the compiler would no longer know how many loads are in flight and would make the
    // wait for A wait for B too); the host passes every vector (replicated scalars, a zero row vector) and only the
    // float bias may be missing, in which case the column term stands in. Every wave leaves its dword in LDS (four
    // waves write the same value to the same place) for the epilogue threads.
    const int t = (int)threadIdx.x;
    int32_t   par_v;
    {
        const int                   v   = wave & 3;
        const int                   j   = min(((int)blockIdx.x + (lane >> 4) * G) * 16 + (lane & 15), g.N - 1);
        const MI355_GLOBAL int32_t *vec = v == 0   ? g_colvec
                                          : v == 1 ? (EPI == EPI_FIXEDPOINT ? g_mult : (EPI == EPI_F32 && has_bias ? g_bias : g_colvec))
                                          : v == 2 ? (EPI == EPI_FIXEDPOINT ? g_shift : g_colvec)
                                                   : g_rowvec;
        par_v                           = vec[v == 3 ? min(lane & (ROWS - 1), g.M - 1) : j];
    }

    // this wave's slice of A: rows past M re-read row M-1 into staging rows whose results are never stored
    char *a_lds = a_stage + wave * ROWS * PITCH;
    v4i   ta[NA];
    const int a_sr = lane / LPR, a_sc = (lane % LPR) * 16;
    // operand blocks of A: lane -> row lane % 16 of a block of rows, 16 bytes at k offset (lane / 16) * 16
    const int arow = lane & 15, akc = (lane >> 4) * 16;
    v4i       fa[RB][PER];
    if constexpr (!A_GLOBAL)
    {
        // lanes past the end of K (last busy wave) re-read the slice's first 16 bytes into columns nobody reads; waves
        // without k blocks re-read the last k block
        const int col = a_sc < min(PER, KB - kb0) * 64 ? a_sc : 0;
#pragma unroll
        for (int i = 0; i < NA; ++i)
            ta[i] = *(const MI355_GLOBAL v4i *)(gA + (int64_t)min(i * RPL + a_sr, g.M - 1) * g.lda + (int64_t)min(kb0, KB - 1) * 64 + col);
    }
    const MI355_GLOBAL int8_t *bp = gB + ((int64_t)min(kb0, KB - 1) * 64 + lane) * 16; // (waves without k blocks re-read the last one)
    // B operand blocks: one group's worth in flight per wave, refilled half by half as the matrix instructions release
    // them; two groups' worth only with a single k block per wave. (Two groups' worth of 4 k blocks fit the registers and
    // were the first design - 128 loads of 1 KiB on offer per compute unit, which admits about 44 - and measured slower:
    // M = 8, N = 11008, K = 4096 9.15 against 8.81 us; M = 16 9.73 / 9.25; M = 32 10.95 / 10.72; N = 32000 22.2 / 21.6;
    // K = 2048 6.17 / 5.95; only K = 1024, one block per wave, prefers two: 4.59 against 4.68 us.)
    constexpr int  H0       = PER / 2;               // k blocks of the first half
    constexpr bool ONE_SLOT = A_GLOBAL || PER >= 2;
    v4i            fb[ONE_SLOT ? 1 : 2][PER];
    auto load_b_part = [&](int slot, int gi, auto u0c, auto u1c)
    {
        const int grp = min((int)blockIdx.x + gi * G, NGT - 1);
#pragma unroll
        for (int u = decltype(u0c)::value; u < decltype(u1c)::value; ++u) // k blocks past KB (last busy wave) re-read the last one
            fb[slot][u] = __builtin_nontemporal_load((const MI355_GLOBAL v4i *)(bp + ((int64_t)grp * KB + max(min(u, KB - 1 - kb0), 0)) * 1024));
    };
    auto load_b = [&](int slot, int gi)
    {
        const int grp = min((int)blockIdx.x + gi * G, NGT - 1);
#pragma unroll
        for (int u = 0; u < PER; ++u)
            fb[slot][u] = __builtin_nontemporal_load((const MI355_GLOBAL v4i *)(bp + ((int64_t)grp * KB + max(min(u, KB - 1 - kb0), 0)) * 1024));
    };
    // MULTI: every workgroup has at least two groups. Nothing between here and the wait for A may sit behind a branch:
    // the compiler would no longer know how many loads are in flight and would make the wait for A wait for B as well
    // (loads return in order) - hence also the unconditional fetches of the epilogue constants below.
    load_b(0, 0);
    __builtin_amdgcn_sched_barrier(0); // group 0 goes out whole before group 1: the first wait then covers group 0 only
    if (MULTI && !ONE_SLOT)
        load_b(1, 1);
    // (with nothing to stage, A is fetched behind the first B blocks: the first matrix instruction needs both anyway,
    // and the stream of B starts that much earlier)
    if constexpr (A_GLOBAL)
    {
        // rows past M re-read row M-1 (never stored), k blocks past KB the last one (set to zero below)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int u = 0; u < PER; ++u)
                fa[rb][u] = *(const MI355_GLOBAL v4i *)(gA + (int64_t)min(rb * 16 + arow, g.M - 1) * g.lda +
                                                        (int64_t)min(kb0 + u, KB - 1) * 64 + akc);
    }
    if constexpr (A_GLOBAL)
    {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int u = 0; u < PER; ++u)
            {
                if (FLIP_A)
                    fa[rb][u] ^= (int)0x80808080;
                if (!(busy && kb0 + u < KB))
                    fa[rb][u] = (v4i){0, 0, 0, 0};
            }
        par[wave & 3][lane] = par_v; // read behind the first group's barrier
    }
    else
    {
#pragma unroll
        for (int i = 0; i < NA; ++i)
        {
            if (FLIP_A)
                ta[i] ^= (int)0x80808080;
            if (i * RPL + a_sr < ROWS && a_sr < RPL)
                *(v4i *)(a_lds + (i * RPL + a_sr) * PITCH + a_sc) = ta[i];
        }
        par[wave & 3][lane] = par_v; // read behind the first group's barrier
        // (rows from ROWS on are zero)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int u = 0; u < PER; ++u)
            {
                fa[rb][u] = (v4i){0, 0, 0, 0};
                if (busy && rb * 16 + arow < ROWS && kb0 + u < KB)
                    fa[rb][u] = *(const v4i *)(a_lds + (rb * 16 + arow) * PITCH + u * 64 + akc);
            }
        if (RED_IN_STAGE)
            __syncthreads(); // every wave has its operands: the staging area becomes the partial results' area
    }

    // The groups of a workgroup, written out for each possible count: with the count a run-time value the fetch of
    // group gi + 2 sits behind a condition, the compiler loses count of the loads in flight, and the matrix instructions
    // of group gi + 1 wait for the loads of group gi + 2 as well.
    auto groups = [&](auto count)
    {
        constexpr int MINE = decltype(count)::value;
#pragma unroll
        for (int gi = 0; gi < MINE; ++gi)
        {
            v4i acc0[RB], acc1[RB < 4 ? RB : 1];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
                acc0[rb] = (v4i){0, 0, 0, 0}, acc1[RB < 4 ? rb : 0] = (v4i){0, 0, 0, 0};
            if (busy)
            {
                // The two chains are added and the sum is held back for 32 issue slots in the same basic block as the
                // matrix instructions: their results may not be read by another instruction type for about a dozen
                // slots, and the compiler only pads that distance inside a block - with the first reader behind a taken
                // branch it came 3 slots after the instruction and read the last register of the result too early.
                if constexpr (ONE_SLOT)
                {
                    // The B blocks of the next group are asked for as soon as their registers are free, half by half.
                    // Four blocks of rows are four independent chains, one accumulator each; fewer blocks alternate
                    // between two accumulators per block like the two-slot form below.
                    auto half = [&](auto u0c, auto u1c)
                    {
#pragma unroll
                        for (int u = decltype(u0c)::value; u < decltype(u1c)::value; ++u)
#pragma unroll
                            for (int rb = 0; rb < RB; ++rb)
                            {
                                if (RB == 4 || !(u & 1))
                                    acc0[rb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[rb][u], fb[0][u], acc0[rb], 0, 0, 0);
                                else
                                    acc1[RB < 4 ? rb : 0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[rb][u], fb[0][u], acc1[RB < 4 ? rb : 0], 0, 0, 0);
                            }
                    };
                    half(std::integral_constant<int, 0>{}, std::integral_constant<int, H0>{});
                    if (gi + 1 < MINE)
                        load_b_part(0, gi + 1, std::integral_constant<int, 0>{}, std::integral_constant<int, H0>{});
                    half(std::integral_constant<int, H0>{}, std::integral_constant<int, PER>{});
                    if (gi + 1 < MINE)
                        load_b_part(0, gi + 1, std::integral_constant<int, H0>{}, std::integral_constant<int, PER>{});
                    if constexpr (RB == 4)
                        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0[0]), "+v"(acc0[1]), "+v"(acc0[2]), "+v"(acc0[3]));
                    else if constexpr (RB == 1)
                    {
                        acc0[0] += acc1[0];
                        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0[0]));
                    }
                    else
                    {
                        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0[0]), "+v"(acc1[0]), "+v"(acc0[RB - 1]), "+v"(acc1[RB - 1]));
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc0[rb] += acc1[RB < 4 ? rb : 0];
                    }
                }
                else
                {
#pragma unroll
                    for (int u = 0; u < PER; ++u)
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            (u & 1 ? acc1[rb] : acc0[rb]) =
                                __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[rb][u], fb[gi & 1][u], u & 1 ? acc1[rb] : acc0[rb], 0, 0, 0);
                    if (RB == 1)
                    {
                        acc0[0] += acc1[0];
                        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0[0]));
                    }
                    else
                    {
                        // (the wait first: the sums below are the first readers of the results)
                        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0[0]), "+v"(acc1[0]), "+v"(acc0[RB - 1]), "+v"(acc1[RB - 1]));
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc0[rb] += acc1[rb];
                    }
                }
            }
            if (!ONE_SLOT && gi + 2 < MINE)
                load_b(gi & 1, gi + 2);
            // accumulator r of lane l is row 4 * (l / 16) + r, column l % 16: lanes 32..63 hold rows 8..15
            if (RL == 64 || lane < 32)
            {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    *(v4i *)&red[((((gi & 1) * WAVES + wave) * RB + rb) * RL + lane) * 4] = acc0[rb];
            }
            __syncthreads();
            // one output per thread and pass (with 64 rows the 512 threads make two passes)
#pragma unroll
            for (int o = t; o < ROWS * 16; o += WAVES * 64)
            {
                // output (erow, ecol): block of rows erow / 16, there accumulator erow % 4 of lane (erow % 16 / 4) * 16 + ecol
                const int      erow = o >> 4, ecol = o & 15;
                const int      j = ((int)blockIdx.x + gi * G) * 16 + ecol;
                const int32_t *r = &red[((((gi & 1) * WAVES) * RB + (erow >> 4)) * RL + ((erow & 15) >> 2) * 16 + ecol) * 4 + (erow & 3)];
                int32_t        sum = 0;
#pragma unroll
                for (int w = 0; w < WAVES; ++w)
                    sum += r[w * RB * RL * 4];
                const int32_t c = par[0][gi * 16 + ecol], m = par[1][gi * 16 + ecol], sh = par[2][gi * 16 + ecol], rv = par[3][erow & (ROWS - 1)];
                if (j < g.N && erow < g.M)
                    once_store_output<EPI>(gD, (int64_t)erow * g.ldd + j, sum, c, m, sh, rv, has_bias, p);
            }
        }
    };
    if (!MULTI || mine == 1)
        groups(std::integral_constant<int, 1>{});
    else if (mine == 2)
        groups(std::integral_constant<int, 2>{});
    else if (mine == 3)
        groups(std::integral_constant<int, 3>{});
    else
        groups(std::integral_constant<int, 4>{});
}
static_assert(ONCE_MAX_GROUPS == 4, "the group loop is written out for 1 to 4 groups");

#undef MI355_GLOBAL

// ---- the stage-once form for deep K: up to 8 rows, 8192 < K <= 16384 -------------------------------------------------
// (the down projection of a transformer's feed-forward block is this shape: few rows, K = 11008 / 14336)
// The same plan - one workgroup of 16 waves per compute unit, every wave stages its K slice of A once and walks the
// column groups - but a wave's slice is NCH chunks of 4 k blocks now, and registers for all of it would leave none for
// B in flight: the operand blocks of A are read from LDS again for every chunk (16 KiB of LDS reads per group and
// workgroup, nothing beside the stream), and B moves in units of one chunk, two units in flight per wave.
#define MI355_GLOBAL __attribute__((address_space(1)))
template <int EPI, bool FLIP_A, int NCH, bool MULTI>
__global__ __launch_bounds__(ONCE_WAVES * 64) void gemm_skinny_deepk_kernel(OnceArgs g)
{
    constexpr int CH = 4, PER = CH * NCH;       // k blocks per chunk / per wave
    constexpr int PPR = PER * 4;                // 16-byte pieces per staged row
    constexpr int PITCH = PER * 64 + 16;        // an odd number of pieces: the 8 rows of an operand read spread over the banks
    constexpr int NA = 8 * PPR / 64;            // staging loads per lane (8 rows)
    __shared__ __attribute__((aligned(16))) int32_t red[2][ONCE_WAVES][32][4];
    __shared__ int32_t                              par[4][64];
    extern __shared__ __attribute__((aligned(16))) char a_stage[]; // [ONCE_WAVES][8][PITCH]

    uintptr_t u_a = (uintptr_t)g.A, u_b = (uintptr_t)g.Bp, u_d = (uintptr_t)g.D, u_cv = (uintptr_t)g.colvec, u_rv = (uintptr_t)g.rowvec,
              u_mu = (uintptr_t)g.mult, u_sh = (uintptr_t)g.shift, u_bf = (uintptr_t)g.bias_f32;
    asm volatile(""
                 : "+s"(g.result_offset), "+s"(g.stage), "+s"(g.lo), "+s"(g.hi), "+s"(g.scale), "+s"(g.act_min), "+s"(g.act_max),
                   "+s"(g.has_offsets), "+s"(g.accumulate), "+s"(g.act_twice), "+s"(g.lda), "+s"(g.ldd), "+s"(g.M), "+s"(g.N),
                   "+s"(g.KB), "+s"(g.grid), "+s"(u_a), "+s"(u_b), "+s"(u_d), "+s"(u_cv), "+s"(u_rv), "+s"(u_mu), "+s"(u_sh),
                   "+s"(u_bf));
    const MI355_GLOBAL int8_t *const  gA = (const MI355_GLOBAL int8_t *)u_a, *const gB = (const MI355_GLOBAL int8_t *)u_b;
    MI355_GLOBAL char *const          gD = (MI355_GLOBAL char *)u_d;
    const MI355_GLOBAL int32_t *const g_colvec = (const MI355_GLOBAL int32_t *)u_cv, *const g_rowvec = (const MI355_GLOBAL int32_t *)u_rv,
                                     *const g_mult = (const MI355_GLOBAL int32_t *)u_mu, *const g_shift = (const MI355_GLOBAL int32_t *)u_sh,
                                     *const g_bias = (const MI355_GLOBAL int32_t *)u_bf;
    const bool has_bias = u_bf != 0;
    EpiParams  p{};
    p.result_offset = g.result_offset, p.stage = g.stage, p.lo = g.lo, p.hi = g.hi;
    p.scale = g.scale, p.act_min = g.act_min, p.act_max = g.act_max;
    p.has_offsets = g.has_offsets, p.accumulate = g.accumulate, p.act_twice = g.act_twice;

    const int t = (int)threadIdx.x, lane = t & 63, wave = t >> 6;
    const int KB = g.KB, NGT = (g.N + 15) / 16, G = g.grid;
    const int mine = (NGT - (int)blockIdx.x + G - 1) / G; // column groups of this workgroup, 1..ONCE_MAX_GROUPS
    const int kb0  = wave * PER;
    const int nb   = min(max(KB - kb0, 0), PER); // k blocks of this wave (the last busy wave may be short, later ones have none)

    // epilogue constants: as in the stage-once kernel (one dword per lane, vector wave % 4, no conditions)
    int32_t par_v;
    {
        const int                   v   = wave & 3;
        const int                   j   = min(((int)blockIdx.x + (lane >> 4) * G) * 16 + (lane & 15), g.N - 1);
        const MI355_GLOBAL int32_t *vec = v == 0   ? g_colvec
                                          : v == 1 ? (EPI == EPI_FIXEDPOINT ? g_mult : (EPI == EPI_F32 && has_bias ? g_bias : g_colvec))
                                          : v == 2 ? (EPI == EPI_FIXEDPOINT ? g_shift : g_colvec)
                                                   : g_rowvec;
        par_v                           = vec[v == 3 ? min(lane & 7, g.M - 1) : j];
    }
    // this wave's slice of A, piece by piece: piece q of the slice is row q / PPR, 16-byte column q % PPR. Rows past M
    // re-read row M-1, columns past the wave's k blocks its first column (neither is ever used)
    char     *a_lds = a_stage + wave * 8 * PITCH;
    v4i       ta[NA];
    const int kbase = min(kb0, KB - 1) * 64;
#pragma unroll
    for (int i = 0; i < NA; ++i)
    {
        const int q = i * 64 + lane, row = q / PPR, pc = q - row * PPR;
        ta[i]       = *(const MI355_GLOBAL v4i *)(gA + (int64_t)min(row, g.M - 1) * g.lda + kbase + (pc < nb * 4 ? pc * 16 : 0));
    }
    // B in units of one chunk of one group: unit c of group gi
    const MI355_GLOBAL int8_t *bp = gB + ((int64_t)min(kb0, KB - 1) * 64 + lane) * 16;
    v4i                        fb[2][CH];
    auto load_unit = [&](int slot, int gi, int c)
    {
        const int grp = min((int)blockIdx.x + gi * G, NGT - 1);
        // (addresses are formed here, unit by unit: hoisted above the dispatch on the number of groups - they are all
        // invariant - the sixteen of them overflow the registers)
        uintptr_t b = (uintptr_t)bp;
        asm volatile("" : "+v"(b));
#pragma unroll
        for (int u = 0; u < CH; ++u) // k blocks past the wave's last re-read it
            fb[slot][u] = __builtin_nontemporal_load(
                (const MI355_GLOBAL v4i *)((const MI355_GLOBAL int8_t *)b + ((int64_t)grp * KB + max(min(c * CH + u, KB - 1 - kb0), 0)) * 1024));
    };
    load_unit(0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_unit(1, 0, 1); // NCH >= 2
#pragma unroll
    for (int i = 0; i < NA; ++i)
    {
        if (FLIP_A)
            ta[i] ^= (int)0x80808080;
        const int q = i * 64 + lane, row = q / PPR, pc = q - row * PPR;
        *(v4i *)(a_lds + row * PITCH + pc * 16) = ta[i];
    }
    par[wave & 3][lane] = par_v; // read behind the first group's barrier
    // operand blocks of A: lane -> row lane % 16 (rows 8..15 are zero), 16 bytes at k offset (lane / 16) * 16
    const int  arow = lane & 15, akc = (lane >> 4) * 16;
    const char *a_rd = a_lds + (arow & 7) * PITCH + akc;
    auto read_a = [&](v4i (&fa)[CH], int c)
    {
#pragma unroll
        for (int u = 0; u < CH; ++u)
        {
            fa[u] = *(const v4i *)(a_rd + (c * CH + u) * 64);
            if (!(arow < 8 && c * CH + u < nb))
                fa[u] = (v4i){0, 0, 0, 0};
        }
    };

    const int erow = t >> 4, ecol = t & 15;
    auto groups = [&](auto count)
    {
        constexpr int MINE = decltype(count)::value;
        v4i fa[2][CH];
        read_a(fa[0], 0);
#pragma unroll
        for (int gi = 0; gi < MINE; ++gi)
        {
            v4i acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < NCH; ++c)
            {
                const int q = gi * NCH + c; // unit in flight order: slot q % 2
                // the operand blocks of A for the next unit, while this unit's B blocks are awaited (read again for every
                // group: without the clobber the compiler keeps all of a wave's blocks in registers, and spills)
                asm volatile("" ::: "memory");
                read_a(fa[(q + 1) & 1], (c + 1) % NCH);
#pragma unroll
                for (int u = 0; u < CH; ++u)
                    (u & 1 ? acc1 : acc0) = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[q & 1][u], fb[q & 1][u], u & 1 ? acc1 : acc0, 0, 0, 0);
                if (q + 2 < MINE * NCH)
                    load_unit(q & 1, (q + 2) / NCH, (q + 2) % NCH);
                __builtin_amdgcn_sched_barrier(0); // units stay apart: moved together, their operands overflow the registers
            }
            // (the sum is held back in the block of the matrix instructions: see the stage-once kernel)
            acc0 += acc1;
            asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc0));
            if (lane < 32)
                *(v4i *)&red[gi & 1][wave][lane][0] = acc0;
            __syncthreads();
            if (t < 128)
            {
                const int      j = ((int)blockIdx.x + gi * G) * 16 + ecol;
                const int32_t *r = &red[gi & 1][0][(erow >> 2) * 16 + ecol][erow & 3];
                int32_t        sum = 0;
#pragma unroll
                for (int w = 0; w < ONCE_WAVES; ++w)
                    sum += r[w * 32 * 4];
                const int32_t c = par[0][gi * 16 + ecol], m = par[1][gi * 16 + ecol], sh = par[2][gi * 16 + ecol], rv = par[3][erow & 7];
                if (j < g.N && erow < g.M)
                    once_store_output<EPI>(gD, (int64_t)erow * g.ldd + j, sum, c, m, sh, rv, has_bias, p);
            }
        }
    };
    if (!MULTI || mine == 1)
        groups(std::integral_constant<int, 1>{});
    else if (mine == 2)
        groups(std::integral_constant<int, 2>{});
    else if (mine == 3)
        groups(std::integral_constant<int, 3>{});
    else
        groups(std::integral_constant<int, 4>{});
}
#undef MI355_GLOBAL

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
static int skinny_launch_v(int epi, bool flip_a, const GemmArgs &a, int batch, hipStream_t s)
{
    const int    groups = (a.N + 15) / 16;
    const dim3   grid((groups + NG - 1) / NG, batch), block(WAVES * 64);
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


// compute units of the current device, asked once per device
int device_cus()
{
    static std::atomic<int> cus[32];
    int                     dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32)
        return 0;
    int n = cus[dev].load(std::memory_order_acquire);
    if (n == 0)
    {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1)
            return 0;
        cus[dev].store(n, std::memory_order_release);
    }
    return n;
}

template <int PER, bool MULTI, int ROWS>
static int skinny_once_launch_r(int epi, bool flip_a, const GemmArgs &a, int grid, hipStream_t s)
{
    constexpr int WAVES = ROWS == 64 ? 8 : ONCE_WAVES;
    static const void *const fns[3][2] = {
        {(const void *)gemm_skinny_once_kernel<EPI_S32, false, PER, MULTI, ROWS, WAVES>,
         (const void *)gemm_skinny_once_kernel<EPI_S32, true, PER, MULTI, ROWS, WAVES>},
        {(const void *)gemm_skinny_once_kernel<EPI_FIXEDPOINT, false, PER, MULTI, ROWS, WAVES>,
         (const void *)gemm_skinny_once_kernel<EPI_FIXEDPOINT, true, PER, MULTI, ROWS, WAVES>},
        {(const void *)gemm_skinny_once_kernel<EPI_F32, false, PER, MULTI, ROWS, WAVES>,
         (const void *)gemm_skinny_once_kernel<EPI_F32, true, PER, MULTI, ROWS, WAVES>}};
    // the kernel fetches these without asking
    if (a.epi.colvec == nullptr || a.epi.rowvec == nullptr || (epi == EPI_FIXEDPOINT && (a.epi.mult == nullptr || a.epi.shift == nullptr)))
        return (int)hipErrorInvalidValue;
    static std::atomic<uint32_t> lds_raised[3][2];
    // staged rows of A; with 32 rows the partial results (2 x 16 waves x 2 blocks x 64 lanes x 16 bytes) share the area
    const size_t                 lds = ROWS == 64 ? (size_t)65536 // nothing staged: only the partial results (2 x 8 waves x 4 blocks)
                                                  : std::max((size_t)ONCE_WAVES * ROWS * once_pitch(ROWS, PER), ROWS > 16 ? (size_t)65536 : (size_t)0);
    const void                  *fn  = fns[epi][flip_a ? 1 : 0];
    // 16 KiB of static LDS on top: declare the dynamic part whatever its size
    const int e = raise_lds_limit(fn, lds, lds_raised[epi][flip_a ? 1 : 0]);
    if (e)
        return e;
    const EpiParams &p = a.epi;
    OnceArgs         o{a.A,    a.Bp,   a.D,    p.colvec, p.rowvec,  p.mult,    p.shift,       p.bias_f32,   a.lda,       a.ldd,        a.M,
               a.N,    (int32_t)(a.Kp / 64), grid, p.result_offset, p.stage, p.lo, p.hi, p.scale, p.act_min, p.act_max,
               p.has_offsets, p.accumulate, p.act_twice};
    void *kargs[] = {&o};
    return (int)hipLaunchKernel(fn, dim3(grid), dim3(WAVES * 64), kargs, lds, s);
}

// (built for one column group per workgroup only: with the group loop written out for 2 to 4 groups as well, the
// compiler's register allocation spills the B blocks as they arrive)
template <int NCH>
static int skinny_deepk_launch(int epi, bool flip_a, const GemmArgs &a, int grid, hipStream_t s)
{
    constexpr bool MULTI = false;
    static const void *const fns[3][2] = {
        {(const void *)gemm_skinny_deepk_kernel<EPI_S32, false, NCH, MULTI>, (const void *)gemm_skinny_deepk_kernel<EPI_S32, true, NCH, MULTI>},
        {(const void *)gemm_skinny_deepk_kernel<EPI_FIXEDPOINT, false, NCH, MULTI>,
         (const void *)gemm_skinny_deepk_kernel<EPI_FIXEDPOINT, true, NCH, MULTI>},
        {(const void *)gemm_skinny_deepk_kernel<EPI_F32, false, NCH, MULTI>, (const void *)gemm_skinny_deepk_kernel<EPI_F32, true, NCH, MULTI>}};
    // the kernel fetches these without asking
    if (a.epi.colvec == nullptr || a.epi.rowvec == nullptr || (epi == EPI_FIXEDPOINT && (a.epi.mult == nullptr || a.epi.shift == nullptr)))
        return (int)hipErrorInvalidValue;
    static std::atomic<uint32_t> lds_raised[3][2];
    const size_t                 lds = (size_t)ONCE_WAVES * 8 * (NCH * 4 * 64 + 16);
    const void                  *fn  = fns[epi][flip_a ? 1 : 0];
    const int                    e   = raise_lds_limit(fn, lds, lds_raised[epi][flip_a ? 1 : 0]);
    if (e)
        return e;
    const EpiParams &p = a.epi;
    OnceArgs         o{a.A,    a.Bp,   a.D,    p.colvec, p.rowvec,  p.mult,    p.shift,       p.bias_f32,   a.lda,       a.ldd,        a.M,
               a.N,    (int32_t)(a.Kp / 64), grid, p.result_offset, p.stage, p.lo, p.hi, p.scale, p.act_min, p.act_max,
               p.has_offsets, p.accumulate, p.act_twice};
    void *kargs[] = {&o};
    return (int)hipLaunchKernel(fn, dim3(grid), dim3(ONCE_WAVES * 64), kargs, lds, s);
}

// 8 k blocks per wave (4096 < K <= 8192): up to 16 rows, whose slices still fit LDS
template <bool MULTI>
static int skinny_once_launch_v8(int epi, bool flip_a, const GemmArgs &a, int grid, hipStream_t s)
{
    return a.M > 8 ? skinny_once_launch_r<8, MULTI, 16>(epi, flip_a, a, grid, s) : skinny_once_launch_r<8, MULTI, 8>(epi, flip_a, a, grid, s);
}

template <int PER, bool MULTI>
static int skinny_once_launch_v(int epi, bool flip_a, const GemmArgs &a, int grid, hipStream_t s)
{
    return a.M > 16  ? skinny_once_launch_r<PER, MULTI, 32>(epi, flip_a, a, grid, s)
           : a.M > 8 ? skinny_once_launch_r<PER, MULTI, 16>(epi, flip_a, a, grid, s)
                     : skinny_once_launch_r<PER, MULTI, 8>(epi, flip_a, a, grid, s);
}

// Workgroups of the stage-once kernels for `groups` column groups on `cus` compute units: one per group while they all
// fit at once; from two groups per unit on, the smallest whole number of workgroups per compute unit that keeps every
// workgroup within ONCE_MAX_GROUPS groups (a grid just above the number of units would leave most of them idle behind
// the first round) - or fewer workgroups with equal shares, see below; in between, half as many workgroups as groups, so that every workgroup still has two (one of them
// three when the count is odd) and no compute unit gets a second workgroup behind its first.
static int once_grid(int groups, int cus)
{
    if (groups <= cus)
        return groups;
    if (groups < 2 * cus)
        return groups / 2;
    // a last round that would occupy an eighth to half of the compute units: the same number of groups for every
    // workgroup, on fewer units, measured 2-7 % faster (a fuller last round, or just a few groups: 0-1 % slower)
    const int r = (groups + cus - 1) / cus, last = groups - (r - 1) * cus;
    if (r <= ONCE_MAX_GROUPS && last >= cus / 8 && last <= cus / 2)
        return (groups + r - 1) / r;
    return cus * ((groups + ONCE_MAX_GROUPS * cus - 1) / (ONCE_MAX_GROUPS * cus));
}

int skinny_launch(int epi, bool flip_a, const GemmArgs &args, int batch, hipStream_t s, const char **variant)
{
    const char *unused;
    const char *&form = variant ? *variant : unused;
    form = "skinny_stream";
    if (args.M < 1 || args.M > SKINNY_MAX_M || args.Kp % 64 != 0 || args.K > args.Kp || batch < 1 || batch > 65535)
        return (int)hipErrorInvalidValue;
    const int groups = (args.N + 15) / 16;
    const int KB     = (int)(args.Kp / 64);
    // Up to 8 rows every wave copies its K slice of A (at most 1 KiB per row) into LDS once and takes its operands
    // from there; that needs nothing to guard
    const bool align_ok = args.K == args.Kp && args.K % 64 == 0 && args.lda % 16 == 0 && ((uintptr_t)args.A & 15) == 0 &&
                          (batch == 1 || args.a_batch_stride % 16 == 0);
    // (a batch along the grid: the streaming form, whose workgroups need nothing from each other)
    const bool align_ok1 = align_ok && batch == 1;
    const bool stage_ok = args.M <= 8 && align_ok;
    const bool once_ok  = args.M <= 32 && align_ok1; // the stage-once form also takes one or two full blocks of 16 rows
    // Up to 4096 of K the stage-once form (grid: once_grid above), each of the 16 waves owning PER = 1, 2 or 4 k blocks;
    // up to 16 rows it also takes 4096 < K <= 8192 with 8 k blocks per wave (one group's worth of B in flight per wave,
    // refilled half by half - the same bytes as two groups of 4 k blocks).
    // up to 8 rows and 8192 < K <= 16384: the stage-once form for deep K (3 or 4 chunks of 4 k blocks per wave)
    if (stage_ok && batch == 1 && KB > 8 * ONCE_WAVES && KB <= 16 * ONCE_WAVES && epi >= EPI_S32 && epi <= EPI_F32)
    {
        const int cus = device_cus();
        if (cus > 0 && groups <= cus) // one column group per workgroup
        {
            form          = "skinny_deepk";
            const int nch = (KB + 4 * ONCE_WAVES - 1) / (4 * ONCE_WAVES);
            return nch == 3 ? skinny_deepk_launch<3>(epi, flip_a, args, groups, s) : skinny_deepk_launch<4>(epi, flip_a, args, groups, s);
        }
    }
    // 33 to 64 rows: the same with 8 waves, each holding the operand blocks of its 1, 2, 4 or 8 k blocks of all 64 rows
    if (args.M > 32 && args.M <= 64 && align_ok1 && KB <= 8 * 8 && epi >= EPI_S32 && epi <= EPI_F32)
    {
        const int cus = device_cus();
        if (cus > 0)
        {
            form             = "skinny_once_64rows";
            const bool multi = groups > cus;
            const int  grid  = once_grid(groups, cus);
            const int  per   = KB <= 8 ? 1 : (KB <= 16 ? 2 : (KB <= 32 ? 4 : 8));
#define MI355_ONCE64(P_)                                                                        \
    (multi ? skinny_once_launch_r<P_, true, 64>(epi, flip_a, args, grid, s)                     \
           : skinny_once_launch_r<P_, false, 64>(epi, flip_a, args, grid, s))
            return per == 1 ? MI355_ONCE64(1) : per == 2 ? MI355_ONCE64(2) : per == 4 ? MI355_ONCE64(4) : MI355_ONCE64(8);
#undef MI355_ONCE64
        }
    }
    if (once_ok && (KB <= 4 * ONCE_WAVES || (KB <= 8 * ONCE_WAVES && args.M <= 16)) && epi >= EPI_S32 && epi <= EPI_F32)
    {
        const int cus = device_cus();
        if (cus > 0)
        {
            form             = "skinny_once";
            const bool multi = groups > cus;
            const int  grid  = once_grid(groups, cus);
            const int  per   = KB <= ONCE_WAVES ? 1 : (KB <= 2 * ONCE_WAVES ? 2 : (KB <= 4 * ONCE_WAVES ? 4 : 8));
            if (per == 8)
                return multi ? skinny_once_launch_v8<true>(epi, flip_a, args, grid, s) : skinny_once_launch_v8<false>(epi, flip_a, args, grid, s);
            if (multi)
                return per == 1   ? skinny_once_launch_v<1, true>(epi, flip_a, args, grid, s)
                       : per == 2 ? skinny_once_launch_v<2, true>(epi, flip_a, args, grid, s)
                                  : skinny_once_launch_v<4, true>(epi, flip_a, args, grid, s);
            return per == 1   ? skinny_once_launch_v<1, false>(epi, flip_a, args, grid, s)
                   : per == 2 ? skinny_once_launch_v<2, false>(epi, flip_a, args, grid, s)
                              : skinny_once_launch_v<4, false>(epi, flip_a, args, grid, s);
        }
    }
    // The kernel lives on loads in flight: 8 waves per workgroup while each of them still has at least one whole
    // step of 8 k blocks and all workgroups are resident together (24 waves of this size per compute unit), 4 otherwise
    int waves = (groups >= 512 && !(stage_ok && KB >= 64 && (int64_t)groups * 8 <= 24 * 256)) ? 4 : 8;
    const int  per   = (KB + waves - 1) / waves;
    const bool stage = stage_ok && per * 64 <= sk_a_slice(waves);
    // more than 8 rows: per-step staging (dword-aligned rows are enough: the staging loads are plain 16-byte loads)
    const bool step = args.M > 8 && args.lda % 4 == 0 && ((uintptr_t)args.A & 3) == 0;
    // (17..24 rows: the gathers of the unstaged variants below re-read row M-1 for the missing rows of the second
    // block, which costs less than staging 32 rows)
    if (args.M > 24 && step)
    {
        // LDS: 8.25 KiB per wave and block of 16 rows; a workgroup covers 2 column groups when there are many
        const int ng     = groups >= 512 ? 2 : 1;
        const int blocks = (groups + ng - 1) / ng;
        if (args.M > 32)
            return ng == 2 ? skinny_launch_v<2, 4, 8, false, 4, true>(epi, flip_a, args, batch, s)
                           : skinny_launch_v<1, 4, 8, false, 4, true>(epi, flip_a, args, batch, s);
        const int w = blocks >= 320 ? 4 : 8;
        if (ng == 2)
            return w == 4 ? skinny_launch_v<2, 4, 8, false, 2, true>(epi, flip_a, args, batch, s)
                          : skinny_launch_v<2, 8, 8, false, 2, true>(epi, flip_a, args, batch, s);
        return w == 4 ? skinny_launch_v<1, 4, 8, false, 2, true>(epi, flip_a, args, batch, s)
                      : skinny_launch_v<1, 8, 8, false, 2, true>(epi, flip_a, args, batch, s);
    }
    if (args.M > 16)
    {
        // More than one block of 16 rows: A (L2 resident) is re-read once per block of the grid, which costs as much as
        // the B stream unless a block covers several column groups - as many as still leave a few hundred blocks.
        const int mr = args.M > 32 ? 4 : 2;
        int       ng = groups >= 1024 ? 4 : (groups >= 512 ? 2 : 1);
        ng = ng >= 4 && mr == 4 ? 4 : (ng >= 2 ? 2 : 1);
        const int blocks = (groups + ng - 1) / ng;
        const int w      = blocks >= 320 ? 4 : 8;
#define MI355_SKV(NG_, MR_)                                                                          \
    (w == 4 ? skinny_launch_v<NG_, 4, 2, false, MR_>(epi, flip_a, args, batch, s)                           \
            : skinny_launch_v<NG_, 8, 2, false, MR_>(epi, flip_a, args, batch, s))
        if (mr == 2)
            return ng == 2 ? MI355_SKV(2, 2) : MI355_SKV(1, 2);
        return ng == 4 ? MI355_SKV(4, 4) : (ng == 2 ? MI355_SKV(2, 4) : MI355_SKV(1, 4));
#undef MI355_SKV
    }
    // the waves of the unstaged / per-step variants follow the old rule
    const int w1 = groups >= 512 ? 4 : 8;
    if (step) // 9..16 rows
        return w1 == 4 ? skinny_launch_v<1, 4, 8, false, 1, true>(epi, flip_a, args, batch, s)
                       : skinny_launch_v<1, 8, 8, false, 1, true>(epi, flip_a, args, batch, s);
    if (stage)
        return waves == 4 ? skinny_launch_v<1, 4, 8, true>(epi, flip_a, args, batch, s) : skinny_launch_v<1, 8, 8, true>(epi, flip_a, args, batch, s);
    return w1 == 4 ? skinny_launch_v<1, 4, 8, false>(epi, flip_a, args, batch, s) : skinny_launch_v<1, 8, 8, false>(epi, flip_a, args, batch, s);
}
} // namespace mi355
