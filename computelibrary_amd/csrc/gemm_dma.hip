// K1 / K4, pipelined variant: the same int8 MFMA GEMM + fused epilogue as gemm_mfma.hip, organised for throughput.
// This is the kernel that runs whenever A rows are 16-byte aligned and K is a multiple of 16; gemm_mfma.hip remains the
// fallback for everything else.
//
// Global -> LDS: direct-to-LDS loads (global_load_lds_dwordx4: no staging registers, no ds_write) into an NS-stage ring,
// so NS-1 K steps of loads are in flight while one is being multiplied. One wave instruction moves 64 lanes x 16 B =
// 1 KiB into consecutive LDS bytes (the hardware adds lane*16 to the LDS base held in M0); a unit therefore covers
// 1024/BK tile rows, and the bank swizzle of mfma_common.hpp is applied on the global side: lane l fetches the 16-byte
// column that belongs at its LDS slot, which stays inside the same BK-byte row segment, so the global access is still
// one contiguous segment per row. The loads are issued from inline assembly with hand-placed s_waitcnt vmcnt(n): the
// compiler cannot tell which stage a direct-to-LDS load writes and would force vmcnt(0) before every LDS read.
//
// Roles: a block has 8 consumer waves and 4 producer waves (3 waves per SIMD). The producers do nothing but issue
// direct-to-LDS loads: such a load occupies its wave for as long as the texture addresser takes to accept it (about 23
// clocks per 1 KiB for the whole compute unit, i.e. about 90 for a wave that shares it with three others), which
// would otherwise stall the wave's matrix instructions. A K step needs (BM + BN) * BK / 1024 of them - for the
// 256 x 128 x 128 tile 48, as many clocks as the step's matrix instructions take - so the addresser must not idle while
// the producers wait in a barrier: for dense tiles the consumers stage the (edge-free, zero-padded) B panel themselves
// in their operand-read slot, and the producers only the A panel.
//
// LDS -> matrix cores: the consumers form two groups of four (one wave of each group per SIMD) that run half a K step
// apart ("ping-pong"): while one group streams its 32 matrix instructions for a K step out of registers, the other
// group reads its operands for the next step from LDS. Two workgroup barriers per K step keep the groups in
// anti-phase; group 1 takes one extra barrier before the loop and group 0 one after it, so every wave executes the
// same number of barriers.
//
// The matrix instruction is v_mfma_i32_16x16x64_i8, not the 32x32x32 one: both do the same multiply-accumulates per
// clock, but the longer K per instruction halves the accumulator updates per multiply, and under this part's power limit
// (random operands) that is worth about 10 % of the kernel's time. Operand traffic is the same: it is set by the wave's
// 64 x 64 sub-tile, 4 + 4 operand blocks of 16 rows x 64 bytes per 64 of K.
//
// Accumulators are kept transposed (the B panel is fed as the first matrix operand), so each lane ends up with 4
// consecutive output columns per accumulator block: the epilogue reads the per-column parameters as 16-byte vectors and
// packs 4 int8 results into one dword. Those dwords go to LDS first (the ring is free by then) and leave as whole
// 128-byte tile rows, 16 bytes per lane; where the destination is not 16-byte aligned they are stored directly.
#include "mfma_common.hpp"

#include <atomic>

namespace mi355
{
__device__ __forceinline__ void dma16(const void *gptr, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory");
}

// scalar-base form: address = sbase (SGPR pair, wave-uniform) + zero-extended per-lane 32-bit offset
__device__ __forceinline__ void dma16s(const void *sbase, uint32_t voff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void block_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Stages the A and B panels of one block tile. All NP producer waves of a block hold one of these. The loads use the
// scalar-base form of the instruction (wave-uniform 64-bit base in SGPRs + one 32-bit offset register per lane): with
// per-lane 64-bit addresses every load costs the SIMD's matrix pipe about 50 clocks, with scalar bases the stream
// overlaps the matrix instructions almost completely. Unit u of a stage (1 KiB = RPU tile rows) belongs to producer
// u % NP. Inside a unit, lane l covers row l / CPR at LDS column slot l % CPR, i.e. global column (l % CPR) ^ swz(row);
// that column is the same for every unit of a wave (see SAME_COL), so a dense producer keeps ONE offset register for A
// and one for B and moves from unit to unit and from K step to K step by scalar additions to the base: no vector
// registers per load (arrays of per-load offsets were spilled to scratch memory, and every reload waited for all the
// loads in flight). Lanes that must read padding instead (K tail of A, out-of-image taps of the implicit convolution)
// need a different base: a wave with any such lane falls back to per-lane addresses for that one load.
template <int BM, int BN, int BK, int NP, int NS, bool CONV>
struct PanelProducer
{
    static constexpr int CPR   = BK / 16;   // 16-byte columns per tile row
    static constexpr int RPU   = 1024 / BK; // tile rows per staging unit (one wave instruction = 1 KiB)
    static constexpr int AU    = BM / RPU;  // staging units of the A part of a stage
    static constexpr int BU    = BN / RPU;
    static constexpr int LPP   = (AU + BU) / NP; // loads per producer wave per stage
    static constexpr int LPA   = (AU + NP - 1) / NP; // at most this many of them are A units
    static constexpr int STAGE = (BM + BN) * BK;
    static_assert((AU + BU) % NP == 0, "staging shape");
    // swz(row) of row = u*RPU + r depends on u only through (u*RPU) & (CPR-1): constant for CPR <= 4, the parity of u
    // for CPR == 8 and u mod 4 for CPR == 16 - and u = pw + i*NP keeps those when NP is a multiple of 2 and 4
    static_assert(CPR <= 4 || (CPR == 8 && NP % 2 == 0) || (CPR == 16 && NP % 4 == 0),
                  "every unit of a producer wave must share the lane -> column map");

    const int8_t *a_base, *b_base, *fill16, *a_end; // wave-uniform
    uint32_t      lane_a, lane_b; // dense A: (l / CPR) * lda + column bytes; B: (l / CPR) * Kp + column bytes
    int           c16;            // byte offset of this lane's column inside a K step
    int           ur;             // this lane's row inside a unit
    int           rows_left;      // M - m0: rows of A at and below the tile's first row
    int64_t       lda, Kp;
    uint32_t      c_off[CONV ? LPA : 1]; // conv: image offset of the (possibly out-of-image) top-left tap of the lane's pixel
    int           c_iy0[CONV ? LPA : 1], c_ix0[CONV ? LPA : 1]; // conv: its input coordinates
    uint32_t      lds0;
    int           pw, K, lane_id;
    int           k_base; // conv: first k of this launch entry's slice of the patch
    ConvGeom      conv;

    __device__ __forceinline__ void init(const GemmArgs &g, int m0, int n0, int bz, int producer_wave, int lane,
                                         uint32_t lds_base)
    {
        pw        = producer_wave;
        lds0      = lds_base;
        K         = g.K;
        k_base    = CONV ? bz * g.k_slice : 0;
        conv      = g.conv;
        fill16    = g.fill16;
        a_end     = g.a_end;
        lane_id   = lane;
        lda       = g.lda;
        Kp        = g.Kp;
        rows_left = g.M - m0;
        a_base    = g.A + (int64_t)bz * g.a_batch_stride + (CONV ? (int64_t)0 : (int64_t)m0 * g.lda);
        b_base    = g.Bp + (int64_t)bz * g.bp_batch_stride + (int64_t)n0 * g.Kp;
        ur        = lane / CPR;
        const int c = (lane % CPR) ^ swz<CPR>(pw * RPU + ur);
        c16       = c * 16;
        lane_a    = (uint32_t)ur * (uint32_t)g.lda + (uint32_t)c16;
        lane_b    = (uint32_t)ur * (uint32_t)g.Kp + (uint32_t)c16;
        if (CONV)
        {
#pragma unroll
            for (int i = 0; i < LPA; ++i)
            {
                const int gr = min(m0 + (pw + i * NP) * RPU + ur, g.M - 1);
                const int t  = fast_div(gr, g.conv.magic_OW);
                const int ox = gr - t * g.conv.OW;
                const int n  = fast_div(t, g.conv.magic_OH);
                const int oy = t - n * g.conv.OH;
                c_iy0[i]     = oy * g.conv.stride_y - g.conv.pad_top;
                c_ix0[i]     = ox * g.conv.stride_x - g.conv.pad_left;
                c_off[i]     = (uint32_t)n * (uint32_t)(g.conv.H * g.conv.W * g.conv.C) +
                           (uint32_t)((c_iy0[i] * g.conv.W + c_ix0[i]) * g.conv.C);
            }
        }
    }

    // The same for a dense tile that lies inside the matrix (no row of it beyond M) and a K step that lies inside K:
    // nothing to decide per load, so the loads go out back to back. (The general form below spends three branches and a
    // dozen scalar instructions on every load; with 12 loads per producer wave and K step that was most of the step.)
    __device__ __forceinline__ void issue_inside(int kt, int slot) const
    {
        static_assert(!CONV, "dense tiles only");
        const uint32_t base = lds0 + (uint32_t)slot * STAGE;
        const int8_t  *a_k  = a_base + (int64_t)kt * BK;
        const int8_t  *b_k  = b_base + (int64_t)kt * BK;
        static_assert(AU % NP == 0, "which panel a load belongs to must not depend on the wave");
#pragma unroll
        for (int i = 0; i < LPP; ++i)
        {
            const int      u   = pw + i * NP; // wave-uniform
            const uint32_t dst = base + (uint32_t)u * 1024u;
            if (i >= AU / NP)
                dma16s(b_k + (int64_t)(u - AU) * RPU * Kp, lane_b, dst);
            else
                dma16s(a_k + (int64_t)u * RPU * lda, lane_a, dst);
        }
    }

    // K step kt of the tile into ring slot `slot`: loads [I0, I1) of this wave's LPP
    template <int I0 = 0, int I1 = LPP>
    __device__ __forceinline__ void issue(int kt, int slot) const
    {
        const int      k0   = kt * BK;
        const uint32_t base = lds0 + (uint32_t)slot * STAGE;
        const int8_t  *a_k  = a_base + (CONV ? 0 : k0);
        const int8_t  *b_k  = b_base + k0; // always inside the zero-padded packed panel
        const bool     full = k0 + BK <= K;
        // convolution: one tap decode per K step (the lane's column is the same in every unit)
        bool     t_in = false;
        int      t_dy = 0, t_dx = 0;
        uint32_t t_off = 0;
        if (CONV)
        {
            const int k   = k_base + k0 + c16; // within the whole patch
            const int tap = fast_div(k, conv.magic_C);
            const int c0  = k - tap * conv.C;
            const int ky  = fast_div(tap, conv.magic_KW);
            const int kx  = tap - ky * conv.KW;
            t_dy          = ky * conv.dil_y;
            t_dx          = kx * conv.dil_x;
            t_off         = (uint32_t)((t_dy * conv.W + t_dx) * conv.C + c0);
            t_in          = k0 + c16 < K;
        }
#pragma unroll
        for (int i = I0; i < I1; ++i)
        {
            const int      u   = pw + i * NP; // wave-uniform
            const uint32_t dst = base + (uint32_t)u * 1024u;
            if (u >= AU)
                dma16s(b_k + (int64_t)(u - AU) * RPU * Kp, lane_b, dst);
            else if (!CONV)
            {
                // rows beyond M re-read row M-1 (their results are never stored): only the last row tile has any
                const bool     edge = (u + 1) * RPU > rows_left;
                const int8_t  *ub   = edge ? a_k : a_k + (int64_t)u * RPU * lda;
                const uint32_t o    = edge ? (uint32_t)min(u * RPU + ur, rows_left - 1) * (uint32_t)lda + (uint32_t)c16 : lane_a;
                if (full)
                    dma16s(ub, o, dst);
                else
                {
                    // last K step. Columns at or beyond K read the fill bytes. A column that straddles K reads on into
                    // the next row (those bytes meet the zero rows of the packed B) - except at the very end of A, where
                    // the lane fetches just the valid bytes and writes its LDS slot itself.
                    const int     k   = k0 + c16;
                    const int8_t *ptr = ub + o;
                    if (k >= K || ptr + 16 <= a_end)
                        dma16(k < K ? ptr : fill16, dst);
                    else
                    {
                        const v4i v = load16_partial(ptr, K - k);
                        *(__attribute__((address_space(3))) v4i *)(size_t)(dst + (uint32_t)lane_id * 16u) = v;
                        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    }
                }
            }
            else
            {
                const int      iy = c_iy0[i < LPA ? i : 0] + t_dy, ix = c_ix0[i < LPA ? i : 0] + t_dx;
                const bool     ok = t_in && (unsigned)iy < (unsigned)conv.H && (unsigned)ix < (unsigned)conv.W;
                const uint32_t o  = c_off[i < LPA ? i : 0] + t_off;
                if (__builtin_amdgcn_ballot_w64(ok) == ~0ull)
                    dma16s(a_k, o, dst);
                else
                    dma16(ok ? a_k + o : fill16, dst);
            }
        }
    }
};

// Measurement build only (-DMI355_PHASE_CLOCKS, a library of its own that the product never loads): the first lane of a
// consumer wave and of a producer wave of three workgroups (first, middle, last) leaves the shader clock counter at the
// ends of the kernel's parts, so that start-up, K loop and epilogue can be told apart without a profiler.
#ifdef MI355_PHASE_CLOCKS
__device__ long long phase_clocks[6][8];
#define MI355_PHASE(i)                                                           \
    do                                                                           \
    {                                                                            \
        if (phase_row >= 0 && lane == 0)                                         \
            phase_clocks[phase_row][i] = (long long)__builtin_readcyclecounter(); \
    } while (0)
#else
#define MI355_PHASE(i) \
    do                 \
    {                  \
    } while (0)
#endif

// GWM x GWN consumer waves per group, 2 groups stacked along M, plus NP = GWM*GWN producer waves
template <int BM, int BN, int BK, int GWM, int GWN, int NS, int EPI, bool FLIP_A, bool CONV>
__global__ __launch_bounds__(GWM *GWN * 192) __attribute__((amdgpu_waves_per_eu(1, 6))) void gemm_dma_kernel(GemmArgs g_in)
{
    // What a workgroup needs before its first loads go out is read here, in one batch of scalar loads, and pinned in
    // registers. Left alone, the compiler fetches kernel arguments where they are first used: five dependent round trips
    // to memory lay between the start of the kernel and its first load. Only scalars and the three pointers of the
    // epilogue constants go through the asm: a pointer that did is generic afterwards, and a generic load waits for LDS
    // and memory alike, so those three come back as pointers to global memory; the operand pointers sit next to pinned
    // scalars in the argument block and arrive with the same loads.
    GemmArgs g = g_in;
    asm volatile(""
                 : "+s"(g.tiles_m), "+s"(g.tiles_n), "+s"(g.magic_tiles), "+s"(g.magic_group), "+s"(g.tile_magic_ok), "+s"(g.lda),
                   "+s"(g.a_batch_stride), "+s"(g.Kp), "+s"(g.bp_batch_stride), "+s"(g.M), "+s"(g.N), "+s"(g.K),
                   "+s"(g.epi.qp_stride), "+s"(g.epi.colvec_batch_stride), "+s"(g.nblocks));
    typedef const __attribute__((address_space(1))) int32_t *global_i32;
    uintptr_t u_cv = (uintptr_t)g.epi.colvec, u_qp = (uintptr_t)g.epi.qp, u_fl = (uintptr_t)g.epi.qp_flag;
    asm volatile("" : "+s"(u_cv), "+s"(u_qp), "+s"(u_fl));
    if (CONV)
        asm volatile(""
                     : "+s"(g.conv.H), "+s"(g.conv.W), "+s"(g.conv.C), "+s"(g.conv.KW), "+s"(g.conv.OW), "+s"(g.conv.OH),
                       "+s"(g.conv.stride_x), "+s"(g.conv.stride_y), "+s"(g.conv.pad_left), "+s"(g.conv.pad_top), "+s"(g.conv.dil_x),
                       "+s"(g.conv.dil_y), "+s"(g.conv.magic_C), "+s"(g.conv.magic_KW), "+s"(g.conv.magic_OW), "+s"(g.conv.magic_OH));

    constexpr int GW    = GWM * GWN; // waves per consumer group
    constexpr int NW    = 2 * GW;    // consumer waves
    constexpr int NP    = GW;        // producer waves (one per SIMD when GW == 4)
    constexpr int CPR   = BK / 16;   // 16-byte columns per tile row
    constexpr int RPU   = 1024 / BK; // tile rows per staging unit
    constexpr int AU = BM / RPU, BU = BN / RPU; // staging units of the A and the B part of a stage
    constexpr int LPP = (AU + BU) / NP;         // loads per producer wave per stage: unit u belongs to producer u % NP
    constexpr int TM = BM / 2 / GWM, TN = BN / GWN;
    constexpr int RS = TM / 16, QS = TN / 16; // 16 x 16 accumulator blocks of a wave: row slots x column slots
    constexpr int KK    = BK / 64;            // matrix instructions along K per stage (each covers 64)
    constexpr int STAGE = (BM + BN) * BK;
    static_assert((AU + BU) % NP == 0, "staging shape");
    // Dense tiles: inside the K loop the consumers stage the B panel themselves (CBU units per wave and K step, issued
    // while their operand reads are in flight) and the producers only the A panel. The block's direct-to-LDS loads then
    // come from all 12 waves instead of 4 and keep flowing while the producers sit in a barrier.
    constexpr bool CDMA = !CONV && (BU % NW == 0) && (AU % NP == 0) && (AU / NP) % 2 == 0;
    constexpr int  CBU  = CDMA ? BU / NW : 0;   // B units per consumer wave per stage
    constexpr int  PLP  = CDMA ? AU / NP : LPP; // loads per producer wave per stage inside the loop
    // Start-up of dense tiles: a wave gets one direct-to-LDS load accepted about every 190 clocks at the start of a kernel,
    // so the first NS-1 stages took the 4 producers 2 x 12 loads = 4.6 k clocks while the consumers sat in barrier 0.
    // All NW + NP waves issue them instead, unit u to wave u % (NW + NP), stage 0 first (4 loads per wave and stage).
    constexpr int  NALL  = NW + NP;
    constexpr int  LPW   = (AU + BU) / NALL; // loads per wave per start-up stage
    constexpr bool SPREAD = CDMA && (AU + BU) % NALL == 0 && (NS - 1) * LPW < 64 &&
                            (CPR <= 4 || (CPR == 8 && NALL % 2 == 0) || (CPR == 16 && NALL % 4 == 0));
    // Small wave tiles: a slot of matrix instructions is much shorter than a slot of operand reads, so running the two
    // consumer groups one slot apart only serialises their reads; both groups then read and multiply in the same slots.
    constexpr bool INPHASE = RS * QS * KK <= 16;
    static_assert(TM % 16 == 0 && TN % 16 == 0 && RS >= 1 && QS >= 1 && BK % 64 == 0, "wave tile");
    static_assert(NS >= 3 && (NS - 2) * LPP < 64, "ring depth / vmcnt range");
    static_assert(NW * 16 * (QS * 64 + 16) <= NS * STAGE, "the 32-bit epilogue stages through the ring's memory");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

#ifdef MI355_PHASE_CLOCKS
    const int phase_blk = blockIdx.x == 0 ? 0 : ((int)blockIdx.x == g.nblocks / 2 ? 1 : ((int)blockIdx.x == g.nblocks - 1 ? 2 : -1));
    const int phase_row = phase_blk < 0 ? -1 : (wave == 0 ? phase_blk * 2 : (wave == NW ? phase_blk * 2 + 1 : -1));
    MI355_PHASE(0); // arguments fetched, first instructions
#endif
    int tm, tn, bz;
    if (g.tile_magic_ok)
        tile_coords_batched_fast(blockIdx.x, g.nblocks, g.tiles_m, g.tiles_n, g.magic_tiles, g.magic_group, bz, tm, tn);
    else
        tile_coords_batched(blockIdx.x, g.nblocks, g.tiles_m, g.tiles_n, bz, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int nk = (g.K + BK - 1) / BK;
    // which requantisation formula applies was decided on the device when the per-column constants were digested
    // (a scalar load: as a vector load its wait would also wait for every direct-to-LDS load issued before it)
    int qflag = 1;
    if (EPI == EPI_FIXEDPOINT && u_fl != 0)
        qflag = *(const __attribute__((address_space(4))) int32_t *)u_fl;
    const bool fast = EPI == EPI_FIXEDPOINT && (qflag & 1) == 0;

    // per-column epilogue constants of this block: fetched now by the consumer waves (before their share of the start-up
    // loads, so that waiting for those covers these too), parked in registers, staged in LDS after the loop
    constexpr int NPAR = (EPI == EPI_FIXEDPOINT) ? 1 + QP_COUNT : 0;
    constexpr int PPT  = (NPAR * BN + NW * 64 - 1) / (NW * 64);
    int32_t       par_reg[PPT > 0 ? PPT : 1];
    if (fast && wave < NW)
    {
#pragma unroll
        for (int t = 0; t < PPT; ++t)
        {
            const int idx = tid + t * NW * 64;
            par_reg[t]    = 0;
            if (idx < NPAR * BN)
            {
                const int par = idx / BN, col = idx % BN;
                par_reg[t]    = par == 0 ? ((global_i32)u_cv)[(int64_t)bz * g.epi.colvec_batch_stride + n0 + col]
                                         : ((global_i32)u_qp)[(int64_t)(par - 1) * g.epi.qp_stride + n0 + col];
            }
        }
    }
    if constexpr (SPREAD)
    {
        PanelProducer<BM, BN, BK, NALL, NS, CONV> first;
        first.init(g, m0, n0, bz, wave, lane, lds0);
#pragma unroll
        for (int s = 0; s < NS - 1; ++s)
            if (s < nk)
                first.issue(s, s % NS);
    }

    // Barrier protocol (b = number of barriers a wave has executed): consumer group 0 reads stage kt between barriers
    // 2kt and 2kt+1 and multiplies it between 2kt+1 and 2kt+2; group 1 does the same one barrier later. Producers make
    // stage kt+1 complete before barrier 2kt+2 and overwrite the ring slot of stage kt-1 after barrier 2kt (its last
    // reader, group 1, finished before that barrier). Every wave executes 2*nk + 2 barriers.
    if (wave >= NW)
    {
        // ================= producer: global -> LDS =================
        PanelProducer<BM, BN, BK, NP, NS, CONV> prod;
        prod.init(g, m0, n0, bz, wave - NW, lane, lds0);
        MI355_PHASE(1); // producer: addresses set up
        if constexpr (!SPREAD)
        {
#pragma unroll
            for (int s = 0; s < NS - 1; ++s)
                if (s < nk)
                    prod.issue(s, s % NS);
        }
        MI355_PHASE(2); // producer: the first NS-1 stages issued
        if (nk >= NS - 1)
            wait_vmcnt<(NS - 2) * (SPREAD ? LPW : LPP)>(); // stage 0 complete, the NS-2 younger stages may still be in flight
        else
            wait_vmcnt<0>();
        MI355_PHASE(3); // producer: its part of stage 0 has landed
        block_barrier(); // barrier 0
        for (int kt = 0; kt < nk; ++kt)
        {
            // A wave gets one direct-to-LDS load accepted about every 90 clocks, so LPP of them take as long as the
            // consumers' whole K step: issue half on either side of the mid-step barrier instead of making both
            // consumer groups wait for all of them. Ring slot of stage kt-1: free since barrier 2kt.
            const bool more = kt + NS - 1 < nk;
            if (more)
                prod.template issue<0, PLP / 2>(kt + NS - 1, (kt + NS - 1) % NS);
            block_barrier(); // barrier 2kt+1
            if (more)
                prod.template issue<PLP / 2, PLP>(kt + NS - 1, (kt + NS - 1) % NS);
            if (more)
                wait_vmcnt<(NS - 2) * PLP>(); // this wave's part of stage kt+1 complete
            else
                wait_vmcnt<0>();
            block_barrier(); // barrier 2kt+2
        }
        block_barrier(); // barrier 2nk+1
        MI355_PHASE(4); // producer: K loop over
        if (fast)
        {
            __syncthreads(); // the consumers' staging of the epilogue constants
            if (g.epi.vec_store16)
                __syncthreads(); // ... and of the output tile
        }
        return;
    }

    // ================= consumers: LDS -> matrix cores =================
    const int group = wave / GW; // waves w and w + GW share a SIMD (waves are placed on the 4 SIMDs round-robin)
    const int wq    = wave % GW;
    const int row_w = group * (BM / 2) + (wq / GWN) * TM; // this wave's sub-tile inside the block tile
    const int col_w = (wq % GWN) * TN;

    v4i acc[RS][QS];
#pragma unroll
    for (int i = 0; i < RS; ++i)
#pragma unroll
        for (int j = 0; j < QS; ++j)
            acc[i][j] = (v4i){0, 0, 0, 0};

    // operand read addresses: lane -> (row lane%16, 16-byte column lane/16) of a 16 row x 64 byte operand block
    const int lr = lane & 15, lh = lane >> 4;
    int       a_rd[RS], b_rd[QS], a_sw[RS], b_sw[QS];
#pragma unroll
    for (int f = 0; f < RS; ++f)
    {
        const int row = row_w + f * 16 + lr;
        a_rd[f]       = row * BK;
        a_sw[f]       = swz<CPR>(row);
    }
#pragma unroll
    for (int f = 0; f < QS; ++f)
    {
        const int row = col_w + f * 16 + lr;
        b_rd[f]       = BM * BK + row * BK;
        b_sw[f]       = swz<CPR>(row);
    }

    // this wave's share of the B panel (CDMA): units wave + i*NW, which all have the lane -> column map of unit `wave`
    const int8_t  *cb_base = g.Bp + (int64_t)bz * g.bp_batch_stride + (int64_t)n0 * g.Kp + (int64_t)wave * RPU * g.Kp;
    const uint32_t cb_lane = (uint32_t)(lane / CPR) * (uint32_t)g.Kp +
                             (uint32_t)(((lane % CPR) ^ swz<CPR>(wave * RPU + lane / CPR)) * 16);
    const uint32_t cb_lds  = lds0 + (uint32_t)(AU + wave) * 1024u;

    MI355_PHASE(1); // consumer: set-up done, waiting for stage 0
    if constexpr (SPREAD)
    {
        // this wave's units of stage 0 (and the epilogue constants before them)
        if (nk >= NS - 1)
            wait_vmcnt<(NS - 2) * LPW>();
        else
            wait_vmcnt<0>();
    }
    block_barrier(); // barrier 0: stage 0 is in LDS
    MI355_PHASE(2); // consumer: stage 0 is in LDS
    if (group == 1 && !INPHASE)
        block_barrier(); // group 1 runs one slot behind group 0

    // row sums of A, taken from the operand blocks as they pass (dense tiles, on request)
    const bool rowsum = !CONV && g.epi.rowsum_mul != 0;
    int32_t    rsum[RS];
#pragma unroll
    for (int f = 0; f < RS; ++f)
        rsum[f] = 0;
    v4i fa[KK][RS], fb[KK][QS];
    for (int kt = 0; kt < nk; ++kt)
    {
        // ---- load slot: operands of K step kt from LDS into registers ----
        const char *s = smem + (kt % NS) * STAGE;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
        {
#pragma unroll
            for (int f = 0; f < RS; ++f)
                fa[kk][f] = *(const v4i *)(s + a_rd[f] + (((kk * 4 + lh) ^ a_sw[f]) << 4));
#pragma unroll
            for (int f = 0; f < QS; ++f)
                fb[kk][f] = *(const v4i *)(s + b_rd[f] + (((kk * 4 + lh) ^ b_sw[f]) << 4));
        }
        if (CDMA && kt + NS - 1 < nk)
        {
            // stage kt+NS-1 goes into the ring slot of stage kt-1, whose last reader finished before barrier 2kt
            const int st = kt + NS - 1;
#pragma unroll
            for (int i = 0; i < CBU; ++i)
                dma16s(cb_base + (int64_t)st * BK + (int64_t)i * NW * RPU * g.Kp, cb_lane,
                       cb_lds + (uint32_t)(st % NS) * STAGE + (uint32_t)(i * NW) * 1024u);
        }
        if (FLIP_A)
        {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                for (int f = 0; f < RS; ++f)
                    fa[kk][f] ^= (int)0x80808080;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (rowsum)
        {
#pragma unroll
            for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                for (int f = 0; f < RS; ++f)
                    rsum[f] = sum_bytes(fa[kk][f], rsum[f]);
        }
        // this wave's units of stage kt+1 have to be in LDS before the barrier that opens that stage to its first
        // reader; the NS-2 younger stages (the last of them just issued) may still be in flight
        if (CDMA)
        {
            if (kt + NS - 1 < nk)
                wait_vmcnt<(NS - 2) * CBU>();
            else
                wait_vmcnt<0>();
        }
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();

        // ---- compute slot: a pure stream of matrix instructions ----
#pragma unroll
        for (int kk = 0; kk < KK; ++kk)
#pragma unroll
            for (int i = 0; i < RS; ++i)
#pragma unroll
                for (int j = 0; j < QS; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[kk][j], fa[kk][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();
    }
    if (CDMA)
        wait_vmcnt<0>();
    if (group == 0 || INPHASE)
        block_barrier(); // barrier 2nk+1; every operand read of every wave is complete beyond this point
    MI355_PHASE(3); // consumer: K loop over
    if (rowsum)
        finish_row_sums<RS>(rsum, g.epi.rowsum_mul, FLIP_A ? nk * BK - g.K : 0);

    if (fast)
    {
        int32_t *par = (int32_t *)smem;
#pragma unroll
        for (int t = 0; t < PPT; ++t)
        {
            const int idx = tid + t * NW * 64;
            if (idx < NPAR * BN)
                par[idx] = par_reg[t];
        }
        __syncthreads();
        if (EPI == EPI_FIXEDPOINT)
        {
            char *stage = smem + ((NPAR * BN * 4 + 15) & ~15);
            const bool rowv = g.epi.rowvec != nullptr || rowsum;
            if (g.epi.vec_store16 && g.epi.qp_std && qflag == 0 && !rowv)
                epilogue_store_staged<true, false, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                       [] { __syncthreads(); });
            else if (g.epi.vec_store16 && g.epi.qp_std && qflag == 0)
                epilogue_store_staged<true, true, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                      [] { __syncthreads(); }, rsum, rowsum);
            else if (g.epi.vec_store16)
                epilogue_store_staged<false, true, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                       [] { __syncthreads(); }, rsum, rowsum);
            else
                epilogue_store_fast<RS, QS, BN>(acc, g, par, m0 + row_w, n0 + col_w, col_w, lane, bz, rsum, rowsum);
        }
    }
    else if ((EPI == EPI_S32 || EPI == EPI_F32) && g.epi.vec_store && !g.epi.accumulate)
    {
        // the ring is free beyond the last barrier: 16 x (QS*64 + 16) bytes per wave
        if constexpr (EPI != EPI_FIXEDPOINT)
            epilogue_store_wave32<EPI, RS, QS>(acc, g, smem + wave * 16 * (QS * 64 + 16), m0 + row_w, n0 + col_w, lane, bz, rsum, rowsum);
    }
    else
        epilogue_store_t<EPI, RS, QS>(acc, g, m0 + row_w, n0 + col_w, lane, bz, rsum, rowsum);
    MI355_PHASE(4); // consumer: epilogue done (stores issued)
}

// The 256 x 128 x 128 tile of a dense GEMM in another division of labour: 4 consumer waves, one per SIMD, in a 2 x 2
// arrangement (wave tile 128 x 64: 8 + 4 operand blocks per 64 of K for 32 matrix instructions, a quarter fewer LDS reads
// than 64 x 64 wave tiles), and 4 producer waves, one per SIMD, that issue every direct-to-LDS load of the block.
// A consumer multiplies one half of a K step (64 deep) out of one register set while the operand reads of the next half
// land in the other set; the reads are interleaved with the first matrix instructions of the half, one read behind each
// instruction, so that after the workgroup barrier - which lets all waves go in the same clock - no wave queues its
// reads in front of its matrix instructions (issued as a block, the reads of all waves kept the matrix pipes empty for
// about 250 clocks per barrier). ONE barrier per K step, in the middle of the step: it opens stage kt+1 to its readers and
// hands the ring slot of stage kt-1 to the producers. Measured against the 8 + 4 wave form above on 2048 x 4096 x 4096:
// 1190 instead of 1640 clocks per K step.
template <int BM, int BN, int BK, int NS, int EPI, bool FLIP_A>
__global__ __launch_bounds__(512) void gemm_wide_kernel(GemmArgs g_in)
{
#ifdef MI355_PHASE_CLOCKS
    const long long t_entry = (long long)__builtin_readcyclecounter(); // before the first argument is asked for
#endif
    GemmArgs g = g_in;
    asm volatile(""
                 : "+s"(g.tiles_m), "+s"(g.tiles_n), "+s"(g.magic_tiles), "+s"(g.magic_group), "+s"(g.tile_magic_ok), "+s"(g.lda),
                   "+s"(g.a_batch_stride), "+s"(g.Kp), "+s"(g.bp_batch_stride), "+s"(g.M), "+s"(g.N), "+s"(g.K),
                   "+s"(g.epi.qp_stride), "+s"(g.epi.colvec_batch_stride), "+s"(g.nblocks));
    typedef const __attribute__((address_space(1))) int32_t *global_i32;
    uintptr_t u_cv = (uintptr_t)g.epi.colvec, u_qp = (uintptr_t)g.epi.qp, u_fl = (uintptr_t)g.epi.qp_flag;
    asm volatile("" : "+s"(u_cv), "+s"(u_qp), "+s"(u_fl));

    constexpr int NW = 4, NP = 4, NALL = NW + NP;
    constexpr int CPR = BK / 16, RPU = 1024 / BK;
    constexpr int AU = BM / RPU, BU = BN / RPU;
    constexpr int LPP = (AU + BU) / NP;   // loads per producer wave per stage
    constexpr int LPW = (AU + BU) / NALL; // loads per wave per start-up stage (all 8 waves issue those)
    constexpr int TM = BM / 2, TN = BN / 2;
    constexpr int RS = TM / 16, QS = TN / 16;
    constexpr int NM = RS * QS, NR = RS + QS; // matrix instructions / operand reads per half step
    constexpr int STAGE = (BM + BN) * BK;
    static_assert(BK == 128, "a K step is two halves of 64");
    static_assert((AU + BU) % NALL == 0 && (NS - 1) * LPW < 64 && (NS - 2) * LPP < 64 && NS >= 3, "staging shape");
    static_assert(NW * 16 * (QS * 64 + 16) <= NS * STAGE, "the 32-bit epilogue stages through the ring's memory");
    static_assert(NM >= NR, "one operand read behind each of the first matrix instructions");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#ifdef MI355_PHASE_CLOCKS
    const int phase_blk = blockIdx.x == 0 ? 0 : ((int)blockIdx.x == g.nblocks / 2 ? 1 : ((int)blockIdx.x == g.nblocks - 1 ? 2 : -1));
    const int phase_row = phase_blk < 0 ? -1 : (wave == 0 ? phase_blk * 2 : (wave == NW ? phase_blk * 2 + 1 : -1));
    MI355_PHASE(0);
    if (phase_row >= 0 && lane == 0)
        phase_clocks[phase_row][5] = t_entry;
#endif
    int tm, tn, bz;
    if (g.tile_magic_ok)
        tile_coords_batched_fast(blockIdx.x, g.nblocks, g.tiles_m, g.tiles_n, g.magic_tiles, g.magic_group, bz, tm, tn);
    else
        tile_coords_batched(blockIdx.x, g.nblocks, g.tiles_m, g.tiles_n, bz, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int nk = (g.K + BK - 1) / BK;
    const bool inside = m0 + BM <= g.M; // no row of this tile lies beyond the matrix
    // which requantisation formula applies was decided on the device when the per-column constants were digested; the
    // word is asked for here and looked at after the first loads have gone out
    int qflag = 1;
    if (EPI == EPI_FIXEDPOINT && u_fl != 0)
        qflag = *(const __attribute__((address_space(4))) int32_t *)u_fl;
    {
        // The first NS-1 stages before anything else - every clock before the first load goes out is a clock in which
        // the whole chip waits for memory: unit u to wave u % 8, stage 0 first
        PanelProducer<BM, BN, BK, NALL, NS, false> first;
        first.init(g, m0, n0, bz, wave, lane, lds0);
#pragma unroll
        for (int s = 0; s < NS - 1; ++s)
            if (s < nk)
            {
                if (inside && (s + 1) * BK <= g.K)
                    first.issue_inside(s, s % NS);
                else
                    first.issue(s, s % NS);
            }
    }
    const bool fast = EPI == EPI_FIXEDPOINT && (qflag & 1) == 0;

    // per-column epilogue constants: fetched by the consumer waves behind their share of the start-up loads, parked in
    // registers, staged in LDS after the loop
    constexpr int NPAR = (EPI == EPI_FIXEDPOINT) ? 1 + QP_COUNT : 0;
    constexpr int PPT  = (NPAR * BN + NW * 64 - 1) / (NW * 64);
    static_assert((NS - 2) * LPW + PPT < 64, "vmcnt range");
    int32_t       par_reg[PPT > 0 ? PPT : 1];
    if (fast && wave < NW)
    {
#pragma unroll
        for (int t = 0; t < PPT; ++t)
        {
            // (every lane loads: the count of loads in flight must not depend on the lane)
            const int idx = min(tid + t * NW * 64, NPAR * BN - 1);
            const int par = idx / BN, col = idx % BN;
            par_reg[t]    = par == 0 ? ((global_i32)u_cv)[(int64_t)bz * g.epi.colvec_batch_stride + n0 + col]
                                     : ((global_i32)u_qp)[(int64_t)(par - 1) * g.epi.qp_stride + n0 + col];
        }
    }

    // Barriers: barrier 0 opens stage 0; barrier kt+1 sits in the middle of K step kt, after every wave's reads of the
    // first half of stage kt were issued ... and completed long before (their data fed the instructions in front of the
    // barrier); it opens stage kt+1 and frees the ring slot of stage kt-1, whose last reads fed matrix instructions that
    // every consumer issued before barrier kt. Every wave executes nk + 2 barriers (+ those of the epilogue).
    if (wave >= NW)
    {
        PanelProducer<BM, BN, BK, NP, NS, false> prod;
        prod.init(g, m0, n0, bz, wave - NW, lane, lds0);
        MI355_PHASE(1);
        MI355_PHASE(2);
        if (nk >= NS - 1)
            wait_vmcnt<(NS - 2) * LPW>();
        else
            wait_vmcnt<0>();
        MI355_PHASE(3);
        block_barrier(); // barrier 0
        // stage kt+NS-1 goes into the slot of stage kt-1: free since barrier kt. A loop of its own for the steps that
        // need no decisions (tile inside the matrix, K step inside K): sharing a loop with the general form, the loads
        // of this one sat between reloads of spilled scalars, and the 12 loads of a producer are the longest chain of a
        // K step.
        int kt = 0;
        if (inside)
        {
            // A last K step that K ends in goes the same way where GemmArgs::lean_tail_bz allows it
            const bool tail_lean = g.lean_tail_bz >= 0 && g.K % BK != 0 && !(bz == g.lean_tail_bz && m0 + BM >= g.M);
            const int  n_lean    = (tail_lean ? nk : g.K / BK) - NS + 1; // steps kt whose stage kt+NS-1 needs no decisions
            for (; kt < n_lean; ++kt)
            {
                prod.issue_inside(kt + NS - 1, (kt + NS - 1) % NS);
                wait_vmcnt<(NS - 2) * LPP>(); // this wave's part of stage kt+1 has landed
                block_barrier();              // barrier kt+1
            }
        }
        for (; kt < nk; ++kt)
        {
            if (kt + NS - 1 < nk)
            {
                prod.issue(kt + NS - 1, (kt + NS - 1) % NS);
                wait_vmcnt<(NS - 2) * LPP>();
            }
            else
                wait_vmcnt<0>();
            block_barrier(); // barrier kt+1
        }
        block_barrier(); // barrier nk+1: every consumer is past its last operand read
        MI355_PHASE(4);
        if (fast)
        {
            __syncthreads(); // the consumers' staging of the epilogue constants
            if (g.epi.vec_store16)
                __syncthreads(); // ... and of the output tile
        }
        return;
    }

    // ================= consumers =================
    const int row_w = (wave >> 1) * TM, col_w = (wave & 1) * TN;
    v4i       acc[RS][QS];
#pragma unroll
    for (int i = 0; i < RS; ++i)
#pragma unroll
        for (int j = 0; j < QS; ++j)
            acc[i][j] = (v4i){0, 0, 0, 0};
    // operand read offsets inside a stage, for the two halves of a K step: lane -> (row lane%16, 16-byte column lane/16)
    const int lr = lane & 15, lh = lane >> 4;
    int       a_rd[2][RS], b_rd[2][QS];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
    {
#pragma unroll
        for (int f = 0; f < RS; ++f)
        {
            const int row = row_w + f * 16 + lr;
            a_rd[kk][f]   = row * BK + (((kk * 4 + lh) ^ swz<CPR>(row)) << 4);
        }
#pragma unroll
        for (int f = 0; f < QS; ++f)
        {
            const int row = col_w + f * 16 + lr;
            b_rd[kk][f]   = BM * BK + row * BK + (((kk * 4 + lh) ^ swz<CPR>(row)) << 4);
        }
    }
    MI355_PHASE(1);
    // this wave's units of stage 0: behind them, stage 1 and the epilogue constants may still be in flight
    if (nk < NS - 1)
        wait_vmcnt<0>();
    else if (fast)
        wait_vmcnt<(NS - 2) * LPW + PPT>();
    else
        wait_vmcnt<(NS - 2) * LPW>();
    block_barrier(); // barrier 0: stage 0 is in LDS
    MI355_PHASE(2);
    v4i fa0[RS], fb0[QS], fa1[RS], fb1[QS];
#pragma unroll
    for (int f = 0; f < RS; ++f)
        fa0[f] = *(const v4i *)(smem + a_rd[0][f]);
#pragma unroll
    for (int f = 0; f < QS; ++f)
        fb0[f] = *(const v4i *)(smem + b_rd[0][f]);
    for (int kt = 0; kt < nk; ++kt)
    {
        const char *s  = smem + (kt % NS) * STAGE;
        const char *s2 = smem + ((kt + 1) % NS) * STAGE; // beyond the last step: whatever the slot holds, never used
        // ---- first half of step kt; the operands of its second half arrive meanwhile ----
#pragma unroll
        for (int f = 0; f < RS; ++f)
            fa1[f] = *(const v4i *)(s + a_rd[1][f]);
#pragma unroll
        for (int f = 0; f < QS; ++f)
            fb1[f] = *(const v4i *)(s + b_rd[1][f]);
        if (FLIP_A)
        {
#pragma unroll
            for (int f = 0; f < RS; ++f)
                fa0[f] ^= (int)0x80808080;
        }

#pragma unroll
        for (int i = 0; i < RS; ++i)
#pragma unroll
            for (int j = 0; j < QS; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb0[j], fa0[i], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < NR; ++r)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // one matrix instruction
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); // one LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NM - NR, 0);
        __builtin_amdgcn_sched_barrier(0);
        // the reads above (second half of stage kt) were issued a dozen matrix instructions ago; they must have left the
        // LDS before the barrier after this one hands their slot to the producers - waiting here costs nothing
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); // (vmcnt: this wave's share of the start-up stages)
        block_barrier(); // barrier kt+1: stage kt+1 is in LDS
        // ---- second half of step kt; the operands of the first half of step kt+1 arrive meanwhile ----
#pragma unroll
        for (int f = 0; f < RS; ++f)
            fa0[f] = *(const v4i *)(s2 + a_rd[0][f]);
#pragma unroll
        for (int f = 0; f < QS; ++f)
            fb0[f] = *(const v4i *)(s2 + b_rd[0][f]);
        if (FLIP_A)
        {
#pragma unroll
            for (int f = 0; f < RS; ++f)
                fa1[f] ^= (int)0x80808080;
        }

#pragma unroll
        for (int i = 0; i < RS; ++i)
#pragma unroll
            for (int j = 0; j < QS; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb1[j], fa1[i], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < NR; ++r)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NM - NR, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
    // the reads issued in the last half step (into fa0 / fb0) are never used, but like every other wave's last operand
    // reads they must have left the LDS before the epilogue writes there
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    block_barrier(); // barrier nk+1
    MI355_PHASE(3);

    if (fast)
    {
        int32_t *par = (int32_t *)smem;
#pragma unroll
        for (int t = 0; t < PPT; ++t)
        {
            const int idx = tid + t * NW * 64;
            if (idx < NPAR * BN)
                par[idx] = par_reg[t];
        }
        __syncthreads();
        if (EPI == EPI_FIXEDPOINT)
        {
            char      *stage = smem + ((NPAR * BN * 4 + 15) & ~15);
            const bool rowv  = g.epi.rowvec != nullptr;
            if (g.epi.vec_store16 && g.epi.qp_std && qflag == 0 && !rowv)
                epilogue_store_staged<true, false, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                       [] { __syncthreads(); });
            else if (g.epi.vec_store16 && g.epi.qp_std && qflag == 0)
                epilogue_store_staged<true, true, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                      [] { __syncthreads(); });
            else if (g.epi.vec_store16)
                epilogue_store_staged<false, true, RS, QS, BM, BN, NW>(acc, g, par, stage, m0, n0, row_w, col_w, wave, lane, bz,
                                                                       [] { __syncthreads(); });
            else
                epilogue_store_fast<RS, QS, BN>(acc, g, par, m0 + row_w, n0 + col_w, col_w, lane, bz);
        }
    }
    else if ((EPI == EPI_S32 || EPI == EPI_F32) && g.epi.vec_store && !g.epi.accumulate)
    {
        if constexpr (EPI != EPI_FIXEDPOINT)
            epilogue_store_wave32<EPI, RS, QS>(acc, g, smem + wave * 16 * (QS * 64 + 16), m0 + row_w, n0 + col_w, lane, bz);
    }
    else
        epilogue_store_t<EPI, RS, QS>(acc, g, m0 + row_w, n0 + col_w, lane, bz);
    MI355_PHASE(4);
}

// ---- instantiation table -------------------------------------------------------------------------------------------
struct DmaEntry
{
    MfmaConfig  cfg;
    int         threads;
    int         lds_bytes;
    const void *fn[3][2][2]; // [epi][flip][conv]
    int         threads_dense = 0; // workgroup size of the dense (non-convolution) kernels when it differs
};

#define MI355_DFN(BM, BN, BK, WM, WN, NS, E, F, C) (const void *)gemm_dma_kernel<BM, BN, BK, WM, WN, NS, E, F, C>
#define MI355_DCFG(NAME, BM, BN, BK, WM, WN, NS)                                                                     \
    {                                                                                                                \
        {NAME, BM, BN, BK}, WM *WN * 192, NS * (BM + BN) * BK,                                                        \
        {                                                                                                            \
            {{MI355_DFN(BM, BN, BK, WM, WN, NS, 0, false, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 0, false, true)}, \
             {MI355_DFN(BM, BN, BK, WM, WN, NS, 0, true, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 0, true, true)}},  \
                {{MI355_DFN(BM, BN, BK, WM, WN, NS, 1, false, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 1, false, true)}, \
                 {MI355_DFN(BM, BN, BK, WM, WN, NS, 1, true, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 1, true, true)}}, \
                {{MI355_DFN(BM, BN, BK, WM, WN, NS, 2, false, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 2, false, true)}, \
                 {MI355_DFN(BM, BN, BK, WM, WN, NS, 2, true, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 2, true, true)}}, \
        }                                                                                                            \
    }

#define MI355_WFN(BM, BN, BK, NS, E, F) (const void *)gemm_wide_kernel<BM, BN, BK, NS, E, F>
// dense: the 4 + 4 wave kernel; convolution: the 8 + 4 wave kernel
#define MI355_WCFG(NAME, BM, BN, BK, WM, WN, NS)                                                                     \
    {                                                                                                                \
        {NAME, BM, BN, BK}, WM *WN * 192, NS * (BM + BN) * BK,                                                        \
        {                                                                                                            \
            {{MI355_WFN(BM, BN, BK, NS, 0, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 0, false, true)},                \
             {MI355_WFN(BM, BN, BK, NS, 0, true), MI355_DFN(BM, BN, BK, WM, WN, NS, 0, true, true)}},                 \
                {{MI355_WFN(BM, BN, BK, NS, 1, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 1, false, true)},            \
                 {MI355_WFN(BM, BN, BK, NS, 1, true), MI355_DFN(BM, BN, BK, WM, WN, NS, 1, true, true)}},             \
                {{MI355_WFN(BM, BN, BK, NS, 2, false), MI355_DFN(BM, BN, BK, WM, WN, NS, 2, false, true)},            \
                 {MI355_WFN(BM, BN, BK, NS, 2, true), MI355_DFN(BM, BN, BK, WM, WN, NS, 2, true, true)}},             \
        },                                                                                                           \
            512                                                                                                      \
    }

// Row sums of A taken inside the kernel (EpiParams::rowsum_mul) are a run-time switch of the 8 + 4 wave kernel; the
// 4 + 4 wave kernel has no registers left for them, so its tile shape falls back to the 8 + 4 wave form there: [epi][flip]
static const void *const g_rowsum_256x128x128[3][2] = {
    {MI355_DFN(256, 128, 128, 2, 2, 3, 0, false, false), MI355_DFN(256, 128, 128, 2, 2, 3, 0, true, false)},
    {MI355_DFN(256, 128, 128, 2, 2, 3, 1, false, false), MI355_DFN(256, 128, 128, 2, 2, 3, 1, true, false)},
    {MI355_DFN(256, 128, 128, 2, 2, 3, 2, false, false), MI355_DFN(256, 128, 128, 2, 2, 3, 2, true, false)}};

static const DmaEntry g_dma[] = {
    MI355_WCFG("pp_256x128x128_s3", 256, 128, 128, 2, 2, 3),
    MI355_DCFG("pp_128x128x128_s3", 128, 128, 128, 2, 2, 3),
    MI355_DCFG("pp_128x64x128_s3", 128, 64, 128, 2, 2, 3),
    MI355_DCFG("pp_64x64x128_s3", 64, 64, 128, 1, 2, 3),
    MI355_DCFG("pp_64x64x128_s6", 64, 64, 128, 1, 2, 6),
    MI355_DCFG("pp_128x64x256_s3", 128, 64, 256, 2, 2, 3),
};

int dma_num_configs()
{
    return (int)(sizeof(g_dma) / sizeof(g_dma[0]));
}
MfmaConfig dma_config(int idx)
{
    MfmaConfig c = g_dma[idx].cfg;
    c.waves      = g_dma[idx].threads / 64;
    c.lds_bytes  = g_dma[idx].lds_bytes;
    return c;
}

int dma_launch(int cfg_idx, int epi, bool flip_a, bool conv, const GemmArgs &args, int batch, hipStream_t s)
{
    if (cfg_idx < 0 || cfg_idx >= dma_num_configs() || epi < 0 || epi > 2)
        return (int)hipErrorInvalidValue;
    const DmaEntry &c  = g_dma[cfg_idx];
    const void     *fn = c.fn[epi][flip_a ? 1 : 0][conv ? 1 : 0];
    int             fn_slot = conv ? 1 : 0; // which entry of the once-per-device table below
    if (args.epi.rowsum_mul != 0)
    {
        if (conv || args.K % 16 != 0)
            return (int)hipErrorInvalidValue;
        if (c.threads_dense) // the 4 + 4 wave kernel's tile shape: see g_rowsum_256x128x128
            fn = g_rowsum_256x128x128[epi][flip_a ? 1 : 0], fn_slot = 2;
    }
    if (fn == nullptr || args.fill16 == nullptr)
        return (int)hipErrorInvalidValue;
    // K slices of a convolution: whole K steps, and K names one slice
    if (args.k_slice != 0 && (!conv || args.K != args.k_slice || args.k_slice % c.cfg.BK != 0 || (int64_t)args.k_slice * batch > args.Kp))
        return (int)hipErrorInvalidValue;
    // shapes the kernel assumes: dword-aligned rows of at least one 16-byte column (whole columns of one tap for the
    // convolution), tiles that cover the output and stay inside the packed B panel
    if (args.K < 16 || args.K > args.Kp || args.Kp % c.cfg.BK != 0 || args.tiles_m * c.cfg.BM < args.M ||
        args.tiles_n * c.cfg.BN < args.N || args.tiles_n * c.cfg.BN > round_up(args.N, PACK_N_ALIGN) || args.M < 1)
        return (int)hipErrorInvalidValue;
    if (conv ? (args.conv.C % 16 != 0 || ((uintptr_t)args.A & 15) != 0 || args.K % 16 != 0)
             : ((((uintptr_t)args.A | (uintptr_t)args.lda | (uintptr_t)args.a_batch_stride) & 3) != 0 || args.a_end == nullptr))
        return (int)hipErrorInvalidValue;
    if (c.lds_bytes > 48 * 1024)
    {
        // once per kernel and device
        static std::atomic<uint32_t> raised[sizeof(g_dma) / sizeof(g_dma[0])][3][2][3];
        std::atomic<uint32_t>       &done = raised[cfg_idx][epi][flip_a ? 1 : 0][fn_slot];
        int                          dev  = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32)
            return (int)hipErrorInvalidDevice;
        if ((done.load(std::memory_order_acquire) & (1u << dev)) == 0)
        {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, c.lds_bytes);
            if (e != hipSuccess)
                return (int)e;
            done.fetch_or(1u << dev, std::memory_order_release);
        }
    }
    GemmArgs a       = args;
    // reciprocals for the tile map: floor(2^32 / d) + 1 gives x / d exactly while x * d < 2^32; the 4-wide groups are
    // split with a 16-bit reciprocal of 3
    const int64_t nblocks = (int64_t)args.tiles_m * args.tiles_n * batch;
    const int64_t d_tiles = (int64_t)args.tiles_m * args.tiles_n, d_group = 4 * (int64_t)args.tiles_n;
    a.tile_magic_ok       = (nblocks * d_tiles < ((int64_t)1 << 32) && d_tiles * d_group < ((int64_t)1 << 32) && d_group < 65536 &&
                       d_tiles > 1 && d_group > 1)
                                ? 1
                                : 0;
    a.magic_tiles = a.tile_magic_ok ? (uint32_t)((((uint64_t)1) << 32) / (uint64_t)d_tiles) + 1u : 0u;
    a.magic_group = a.tile_magic_ok ? (uint32_t)((((uint64_t)1) << 32) / (uint64_t)d_group) + 1u : 0u;
    a.nblocks     = (int32_t)nblocks;
    // (rows and batch entries at least a K step apart: what a whole last step reads beyond K then lies in the next row or
    // entry, in front of a_end; not when the kernel sums the rows of A from the same tiles)
    a.lean_tail_bz = (!conv && args.K % c.cfg.BK != 0 && args.epi.rowsum_mul == 0 && args.lda >= c.cfg.BK &&
                      (batch == 1 || args.a_batch_stride >= c.cfg.BK))
                         ? batch - 1
                         : -1;
    void    *kargs[] = {&a};
    dim3     grid(args.tiles_m * args.tiles_n * batch, 1, 1), block((fn_slot == 0 && c.threads_dense) ? c.threads_dense : c.threads);
    return (int)hipLaunchKernel(fn, grid, block, kargs, c.lds_bytes, s);
}
} // namespace mi355

#ifdef MI355_PHASE_CLOCKS
// 6 rows (first / middle / last workgroup x consumer wave 0, producer wave 0) of 8 clock readings, of the last launch
extern "C" int mi355_phase_clocks_read(long long *out)
{
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(mi355::phase_clocks), sizeof(long long) * 48);
}
#endif
