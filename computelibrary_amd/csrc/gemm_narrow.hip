// K5: implicit-GEMM convolution (and dense GEMM) with few output columns: N <= 64, K <= 1152 - or, with K <= 192, up to
// 256 columns as 2 to 4 panels of 64 (a 1 x 1 convolution that widens few channels: the patch of a wave stays in its
// registers and goes against one panel after the other, every panel with its own epilogue).
//
// CpuGemmConv2d lowers a convolution with 64 output channels to a GEMM with M = batch * OH * OW rows and 64 columns
// (src/cpu/operators/CpuGemmConv2d.cpp:923-1008); the work per output tile is then so small (K = KH * KW * C) that a
// tile kernel built around a ring of K steps spends its time on start-up, barriers and epilogues. Here nothing is
// shared between waves but the weights:
//   * the whole B panel (64 columns x K, K contiguous, from the packed Bp) is copied into LDS once per workgroup, rows
//     padded by 16 bytes so that the 16 rows of an operand read fall into 16 different bank groups;
//   * every wave owns 32 output rows x all 64 columns and fetches its A operands straight from global memory into the
//     matrix cores' operand layout - lane l holds 16 bytes of row l % 16 at k offset (l / 16) * 16, for NHWC with
//     C % 16 == 0 that is 16 channels of one tap of one pixel, so a wave load covers whole pixels, and every A byte is
//     used against all 64 columns out of registers;
//   * loads go out in batches of 3 k blocks (6 loads of 1 KiB per wave), two batches in flight, and the number of
//     batches is a template parameter, so the code is straight-line and the compiler knows exactly how many loads
//     are outstanding at every wait;
//   * the A loads are buffer loads with the hardware's range check (a tap above the first or below the last image row
//     lies outside the tensor and reads as zero without a test), so a load costs one addition; which pieces are padding
//     is worked out after the loads have been issued, while they are in flight;
//   * no barrier after the one that publishes the B panel; 4 workgroups of 4 waves fit a compute unit.
#include "mfma_common.hpp"

#include <algorithm>
#include <atomic>
#include <type_traits>

namespace mi355
{
// global -> LDS without registers: 64 lanes x 16 bytes land at M0 + lane * 16
// (scalar base + one 32-bit offset per lane)
__device__ __forceinline__ void narrow_dma16(const void *sbase, uint32_t voff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}
// (one 64-bit address per lane)
__device__ __forceinline__ void narrow_dma16_at(const void *from, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(from), "s"(lds_addr) : "memory");
}

// x / d with the reciprocal of ConvGeom::magic_* (0 stands for d == 1), without a branch on the reciprocal
__device__ __forceinline__ int narrow_div(int x, uint32_t magic)
{
    const uint32_t one = (uint32_t)(magic != 0) - 1u; // all ones when d == 1
    return (int)(__umulhi((uint32_t)x, magic) + ((uint32_t)x & one));
}

// bitwise OR of x over the 64 lanes of the wave, as a scalar
__device__ __forceinline__ uint32_t wave_or(uint32_t x)
{
    // row_shr within rows of 16 lanes (bound_ctrl: lanes without a source read 0), then the four row results
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, true); // row_shr:1
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, true); // row_shr:2
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, true); // row_shr:4
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, true); // row_shr:8
    // lane 15 of every row now holds the row's OR
    return (uint32_t)__builtin_amdgcn_readlane((int)x, 15) | (uint32_t)__builtin_amdgcn_readlane((int)x, 31) |
           (uint32_t)__builtin_amdgcn_readlane((int)x, 47) | (uint32_t)__builtin_amdgcn_readlane((int)x, 63);
}

constexpr int NARROW_WAVES  = 4;
constexpr int NARROW_ROWS   = 32;  // per wave
constexpr int NARROW_BN     = 64;
constexpr int NARROW_MAX_NB = 6;   // batches of 3 k blocks of 64: K <= 1152
constexpr int NARROW_MAX_PANELS = 4; // panels of 64 columns with one batch (K <= 192): N <= 256 (8 panels fill LDS with one
                                     // workgroup's weights and measured slower than the tiled kernel)

// UNI: C % 64 == 0 - a k block of 64 lies inside one tap, so the tap of a load is decoded with scalar arithmetic
template <int EPI, bool FLIP_A, bool CONV, bool UNI, int NB>
// (4 waves per SIMD, i.e. 4 workgroups per compute unit: at most 128 registers per lane)
__global__ __launch_bounds__(NARROW_WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_narrow_kernel(GemmArgs g)
{
    constexpr int RS = NARROW_ROWS / 16, QS = NARROW_BN / 16;
    constexpr int KBLK  = NB * 3;         // k blocks the loop covers (the B panel is zero beyond K)
    constexpr int PITCH = KBLK * 64 + NARROW_PAD_PIECES * 16; // bytes per B row in LDS
    constexpr int NPAR  = 1 + QP_COUNT;
    extern __shared__ __attribute__((aligned(16))) char smem[]; // B panel [npan * 64][PITCH], then par[NPAR][npan * 64]

    // Everything the main part uses is fetched here in one batch of scalar loads and pinned in registers (left alone, the
    // compiler fetches kernel arguments where they are first used: a round trip to memory each time). Pointers go
    // through the asm as integers and come back as pointers to global memory.
#define MI355_GLOBAL __attribute__((address_space(1)))
    ConvGeom  cg = g.conv;
    uintptr_t u_a = (uintptr_t)g.A, u_b = (uintptr_t)g.Bp, u_cv = (uintptr_t)g.epi.colvec, u_qp = (uintptr_t)g.epi.qp,
              u_fl = (uintptr_t)g.epi.qp_flag;
    uint32_t  a_bytes = (uint32_t)(g.a_end - g.A); // bytes of A: what the range check of the A loads compares with
    int32_t   a_M = g.M, a_K = g.K, a_lda = (int32_t)g.lda, a_kp = (int32_t)g.Kp, a_qps = (int32_t)g.epi.qp_stride;
    int32_t   tail_start = g.tiles_m, tail_waves = g.tiles_n; // see narrow_launch
    int32_t   a_npan = g.nblocks;                             // panels of 64 columns (more than one only with NB == 1)
    asm volatile(""
                 : "+s"(cg.H), "+s"(cg.W), "+s"(cg.C), "+s"(cg.KW), "+s"(cg.OW), "+s"(cg.OH), "+s"(cg.stride_x), "+s"(cg.stride_y),
                   "+s"(cg.pad_left), "+s"(cg.pad_top), "+s"(cg.dil_x), "+s"(cg.dil_y), "+s"(cg.pad_word), "+s"(cg.magic_C),
                   "+s"(cg.magic_KW), "+s"(cg.magic_OW), "+s"(cg.magic_OH), "+s"(a_M), "+s"(a_K), "+s"(a_lda), "+s"(a_kp),
                   "+s"(a_qps), "+s"(u_a), "+s"(u_b), "+s"(u_cv), "+s"(u_qp), "+s"(u_fl), "+s"(a_bytes), "+s"(tail_start), "+s"(tail_waves),
                   "+s"(a_npan));
    const int npan = NB == 1 ? a_npan : 1; // (a constant for the deeper forms: their code does not change)
    const int BNT  = npan * NARROW_BN;     // columns in LDS
    int32_t  *par  = (int32_t *)(smem + BNT * PITCH);
    const MI355_GLOBAL int8_t *const gB = (const MI355_GLOBAL int8_t *)u_b;
    // raw buffer over A (stride 0, 32-bit elements untyped): loads at or past a_bytes - also "negative" offsets, which
    // are huge as unsigned - return zero
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)u_a, 0, (int)a_bytes, 0x00020000);
    const MI355_GLOBAL int32_t *const g_colvec = (const MI355_GLOBAL int32_t *)u_cv, *const g_qp = (const MI355_GLOBAL int32_t *)u_qp;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lh = lane >> 4;
    // Workgroups from tail_start on cover only tail_waves * 32 rows each (their other waves help with the B panel and
    // leave): the last, partial round of workgroups is spread over more compute units in smaller pieces.
    const int  tail   = (int)blockIdx.x - tail_start;
    const int  row0   = tail < 0 ? (int)blockIdx.x * (NARROW_WAVES * NARROW_ROWS) + wave * NARROW_ROWS
                                 : tail_start * (NARROW_WAVES * NARROW_ROWS) + (tail * tail_waves + wave) * NARROW_ROWS;
    const bool active = (tail < 0 || wave < tail_waves) && row0 < a_M;

    // the epilogue's per-column constants (column term + the digested requantisation vectors), where they exist: 6 x 64
    // dwords, one or two per thread, fetched first and parked in LDS with the B panel
    const bool    have_qp = EPI == EPI_FIXEDPOINT && u_qp != 0;
    constexpr int TPN     = NB == 1 ? (NPAR * NARROW_BN * NARROW_MAX_PANELS + NARROW_WAVES * 64 - 1) / (NARROW_WAVES * 64) : 2; // dwords per thread
    int32_t       tp[TPN];
#pragma unroll
    for (int i = 0; i < TPN; ++i)
        tp[i] = 0;
    if (have_qp)
    {
#pragma unroll
        for (int i = 0; i < TPN; ++i)
        {
            if (NB == 1 && i * NARROW_WAVES * 64 >= NPAR * BNT) // (wave-uniform)
                break;
            const int idx = min(tid + i * NARROW_WAVES * 64, NPAR * BNT - 1);
            const int v = idx / BNT, col = idx - v * BNT;
            tp[i]       = v == 0 ? g_colvec[col] : g_qp[(v - 1) * a_qps + col];
        }
    }
    auto park_constants = [&]()
    {
        if (!have_qp)
            return;
#pragma unroll
        for (int i = 0; i < TPN; ++i)
            if (tid + i * NARROW_WAVES * 64 < NPAR * BNT)
                par[tid + i * NARROW_WAVES * 64] = tp[i];
    };
    int qflag = 1;
    if (have_qp && u_fl != 0)
        qflag = *(const MI355_GLOBAL int32_t *)u_fl;

    // ---- B panel: straight into LDS (no registers), issued before the A loads, which are needed later. The host keeps
    // the panel in global memory exactly as it lies in LDS (rows of CHUNKS pieces of 16 bytes plus NARROW_PAD_PIECES of padding,
    // zero beyond Kp), so it moves as NDMA linear transfers of 1 KiB; wave w issues transfers w, w + 4, ... ----
    constexpr int  CHUNKS = KBLK * 4;       // 16-byte pieces of a row that hold data
    constexpr int  NDMA   = CHUNKS + NARROW_PAD_PIECES; // 64 rows x that many pieces / 64 pieces per transfer
    constexpr int  DPW    = (NDMA + NARROW_WAVES - 1) / NARROW_WAVES;
    const uint32_t lds0   = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;
    if (NB == 1)
    {
        // (any number of panels: a loop)
        for (int ins = wave; ins < npan * NDMA; ins += NARROW_WAVES)
            narrow_dma16((const void *)(gB + ins * 1024), (uint32_t)lane * 16u, lds0 + (uint32_t)ins * 1024u);
    }
    else
    {
#pragma unroll
        for (int i = 0; i < DPW; ++i)
        {
            const int ins = wave + i * NARROW_WAVES;
            if (ins < NDMA)
                narrow_dma16((const void *)(gB + ins * 1024), (uint32_t)lane * 16u, lds0 + (uint32_t)ins * 1024u);
        }
    }

    if (!active)
    {
        // this wave's share of the B panel and of the constants, then out
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        park_constants();
        __syncthreads();
        return;
    }

    // ---- A: per-lane source of row rb*16 + lr ----
    // conv: pix[rb] = byte offset of the (possibly out-of-image) top-left tap of the row's pixel, iy0/ix0 its coordinates;
    // dense: byte offset of the row. Rows past M re-use row M-1 (never stored).
    int32_t pix[RS], iy0[RS], ix0[RS];
#pragma unroll
    for (int rb = 0; rb < RS; ++rb)
    {
        const int gr = min(row0 + rb * 16 + lr, a_M - 1);
        if (CONV)
        {
            const int t  = narrow_div(gr, cg.magic_OW);
            const int ox = gr - t * cg.OW;
            const int n  = narrow_div(t, cg.magic_OH);
            const int oy = t - n * cg.OH;
            iy0[rb]      = oy * cg.stride_y - cg.pad_top;
            ix0[rb]      = ox * cg.stride_x - cg.pad_left;
            pix[rb]      = n * (cg.H * cg.W * cg.C) + (iy0[rb] * cg.W + ix0[rb]) * cg.C;
        }
        else
        {
            iy0[rb] = ix0[rb] = 0;
            pix[rb]           = gr * a_lda;
        }
    }
    // A piece outside the image is replaced by the padding value when it is used; its load goes out all the same (inside
    // the tensor it reads a neighbouring pixel, outside it reads zero). Past K the value is irrelevant: B is zero there.
    v4i      fa[2][3][RS];
    uint32_t oob = 0;      // bit (slot * 3 + kk) * RS + rb: that piece is padding
    uint32_t oob_wave = 0; // the same bits, set where any lane of the wave has them set (scalar: most pieces of most
                           // waves have nothing to replace, and a scalar test skips them without vector work)
    // tap of k block kb (UNI: scalar) or of this lane's 16 bytes of it
    auto tap_of = [&](int kb, int &dy, int &dx, int &off)
    {
        const int k = kb * 64 + lh * 16;
        dy = 0, dx = 0, off = k;
        if (CONV)
        {
            int tap, c0;
            if (UNI)
            {
                tap = narrow_div(kb * 64, cg.magic_C); // scalar
                c0  = kb * 64 - tap * cg.C + lh * 16;
            }
            else
            {
                tap = narrow_div(k, cg.magic_C);
                c0  = k - tap * cg.C;
            }
            const int ky = narrow_div(tap, cg.magic_KW);
            const int kx = tap - ky * cg.KW;
            dy           = ky * cg.dil_y;
            dx           = kx * cg.dil_x;
            off          = (dy * cg.W + dx) * cg.C + c0;
        }
    };
    auto load_a = [&](int slot, int batch)
    {
#pragma unroll
        for (int kk = 0; kk < 3; ++kk)
        {
            int dy, dx, off;
            tap_of(batch * 3 + kk, dy, dx, off);
#pragma unroll
            for (int rb = 0; rb < RS; ++rb)
                fa[slot][kk][rb] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(a_rsrc, pix[rb] + off, 0, 0);
        }
    };
    auto mask_a = [&](int slot, int batch)
    {
        if (!CONV)
            return;
        oob &= ~(((1u << (3 * RS)) - 1u) << (slot * 3 * RS));
#pragma unroll
        for (int kk = 0; kk < 3; ++kk)
        {
            int dy, dx, off;
            tap_of(batch * 3 + kk, dy, dx, off);
#pragma unroll
            for (int rb = 0; rb < RS; ++rb)
            {
                const bool ok = ((unsigned)(iy0[rb] + dy) < (unsigned)cg.H) & ((unsigned)(ix0[rb] + dx) < (unsigned)cg.W);
                oob |= (uint32_t)(!ok) << ((slot * 3 + kk) * RS + rb);
            }
        }
        oob_wave = wave_or(oob);
    };
    load_a(0, 0);
    if (NB > 1)
        load_a(1, 1);
    __builtin_amdgcn_sched_barrier(0); // nothing else moves up between the loads: they go out first
    mask_a(0, 0);
    if (NB > 1)
        mask_a(1, 1);

    // ---- the B panel has landed when at most the A loads issued after it are still in flight; epilogue constants ----
    if (NB > 1)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * 3 * RS) : "memory");
    else
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * RS) : "memory");
    park_constants();
    qflag           = __builtin_amdgcn_readfirstlane(qflag);
    const bool fast = have_qp && (qflag & 1) == 0;
    __syncthreads();

    // The waves of a SIMD would otherwise share the matrix pipe evenly, finish together and then all queue for the vector
    // ALU with their epilogues: different priorities let one wave at a time through the matrix instructions, and its
    // epilogue then runs beside the matrix instructions of the next.
    // (workgroups go to the 8 XCDs round-robin: those that meet on a compute unit differ in the bits above the low three)
    switch ((blockIdx.x >> 3) & 3)
    {
    case 0: __builtin_amdgcn_s_setprio(3); break;
    case 1: __builtin_amdgcn_s_setprio(2); break;
    case 2: __builtin_amdgcn_s_setprio(1); break;
    default: break;
    }
    // one panel of 64 columns after the other against the same patch (more than one panel: NB == 1, the whole patch is
    // in fa[0]); every panel has its own accumulators and epilogue
    for (int np = 0; np < npan; ++np)
    {
    const int col0 = np * NARROW_BN;
    v4i       acc[RS][QS];
#pragma unroll
    for (int i = 0; i < RS; ++i)
#pragma unroll
        for (int j = 0; j < QS; ++j)
            acc[i][j] = (v4i){0, 0, 0, 0};
    const char *b_rd = smem + (col0 + lr) * PITCH + lh * 16; // + q * 16 * PITCH + kb * 64
#pragma unroll
    for (int b = 0; b < NB; ++b)
    {
#pragma unroll
        for (int kk = 0; kk < 3; ++kk)
        {
            // (a single batch that K does not fill, K = 64 or 128 under many columns: the k blocks past K hold zeros in
            // the panel - skip them, every panel would multiply them again)
            if (NB == 1 && kk > 0 && kk * 64 >= a_K)
                continue;
            v4i fb[QS];
#pragma unroll
            for (int q = 0; q < QS; ++q)
                fb[q] = *(const v4i *)(b_rd + q * 16 * PITCH + (b * 3 + kk) * 64);
#pragma unroll
            for (int rb = 0; rb < RS; ++rb)
            {
                v4i a = fa[b & 1][kk][rb];
                if (CONV && (oob_wave & (1u << (((b & 1) * 3 + kk) * RS + rb))))
                {
                    // (the asm keeps this a branch - as selects it would cost every wave four instructions per piece -
                    // and puts two idle cycles between the vector writes and the matrix instruction that reads them)
                    if (oob & (1u << (((b & 1) * 3 + kk) * RS + rb)))
                        a = (v4i){(int)cg.pad_word, (int)cg.pad_word, (int)cg.pad_word, (int)cg.pad_word};
                    asm volatile("s_nop 1" : "+v"(a));
                }
                if (FLIP_A)
                    a ^= (int)0x80808080;
#pragma unroll
                for (int q = 0; q < QS; ++q)
                    acc[rb][q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[q], a, acc[rb][q], 0, 0, 0);
            }
        }
        if (b + 2 < NB)
        {
            load_a(b & 1, b + 2);
            mask_a(b & 1, b + 2);
        }
    }

    __builtin_amdgcn_s_setprio(0);
    if (fast && g.epi.qp_std && (qflag & 3) == 0 && g.epi.vec_store && (g.N & 3) == 0)
    {
        // every column has a normalised multiplier and a right shift of 2..31: the short form of the requantisation.
        // Lane l holds, for row rb * 16 + l % 16, the 4 consecutive columns q * 16 + 4 * (l / 16) + {0..3}: one dword
        // (N is a multiple of 4 here, so a lane's four columns exist together or not at all).
        const int32_t  off2p1 = 2 * g.epi.result_offset + 1, lo = g.epi.lo, hi = g.epi.hi;
        const int32_t *rowvec = g.epi.rowvec;
        const int      a_N    = g.N;
        int32_t        rv[RS];
        char          *drow[RS]; // this lane's row of D at column 4 * (l / 16)
#pragma unroll
        for (int rb = 0; rb < RS; ++rb)
        {
            const int i = row0 + rb * 16 + lr;
            rv[rb]      = (rowvec && i < a_M) ? rowvec[i] : 0;
            drow[rb]    = (char *)g.D + (int64_t)i * g.ldd + col0 + 4 * lh;
        }
#pragma unroll
        for (int q = 0; q < QS; ++q)
        {
            const int c  = q * 16 + 4 * lh;
            const v4i s2 = *(const v4i *)(par + (1 + QP_S2) * BNT + col0 + c), r1 = *(const v4i *)(par + (1 + QP_RSM1) * BNT + col0 + c);
            const v4i cv = *(const v4i *)(par + col0 + c);
#pragma unroll
            for (int rb = 0; rb < RS; ++rb)
            {
                int32_t o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t)
                {
                    // std_requant with the clamp as one median instruction (lo <= hi)
                    const int32_t v = (int32_t)((uint32_t)acc[rb][q][t] + (uint32_t)cv[t] + (uint32_t)rv[rb]);
                    const int32_t h = __mulhi(v, s2[t]) + v;
                    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(o[t]) : "v"(((h >> r1[t]) + off2p1) >> 1), "s"(lo), "v"(hi));
                }
                const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)o[1], (uint32_t)o[0], 0x0c0c0400u);
                const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)o[3], (uint32_t)o[2], 0x0c0c0400u);
                if (row0 + rb * 16 + lr < a_M && col0 + c < a_N)
                    *(uint32_t *)(drow[rb] + q * 16) = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
            }
        }
    }
    else if (fast && npan == 1)
        epilogue_store_fast<RS, QS, NARROW_BN>(acc, g, par, row0, 0, 0, lane, 0);
    else
        epilogue_store_t<EPI, RS, QS>(acc, g, row0, col0, lane, 0);
    }
#undef MI355_GLOBAL
}

// ---- the same convolution for large images: the input rows a workgroup needs, staged once in LDS ---------------------
// Above, every wave fetches its 32 patches tap by tap from global memory: KH * KW times the image crosses the compute
// unit's vector-memory path (one 1 KiB load instruction every 20 clocks or so, whatever the caches hold), and with more
// than a few tiles per compute unit that path, not the matrix cores, sets the time (config 4 of the benchmark: 327 KiB
// per compute unit = 3 us of an 8.5 us kernel, and 1.9 us more for the B panel that each of its three workgroups
// copies). Here ONE workgroup of 16 waves takes a band of output rows of one image: the window of input rows and
// columns under the band (band + halo + padding) is copied into LDS once, next to the one B panel, by direct-to-LDS
// loads - a lane of a transfer fetches 16 bytes of a pixel, or 16 bytes of the padding value where the window leaves the
// image; the 16-byte pieces of a pixel are permuted so that the 16 pixels of an operand read fall into 16 bank groups -
// and every wave forms the operand blocks of its 32 output pixels with per-lane LDS addresses: a tap is a shift of the
// pixel index, no test. (With the tests and a select per tap and row the kernel was bound by the vector ALU, not by
// the matrix cores or LDS: 700 issue slots per wave, a third of them in the k loop.)
// Needs C a power of two >= 64 (a 64-byte k block then lies inside one tap and one pixel), N <= 64, K <= 1152.
constexpr int HALO_WAVES = 16;
constexpr int HALO_DMA_WAVES = 8; // waves that issue the window's transfers
// ... and the panel's: every wave - these go out in front of the argument fetch, which the last waves wait for longest
// (0.1 us faster than from the first 8 waves only)
constexpr int HALO_PANEL_WAVES = HALO_WAVES;

// Measurement build only (-DMI355_PHASE_CLOCKS, a library of its own that the product never loads): the first lane of
// wave 0 and of wave 12 of the first, the middle and the last workgroup leaves the 100 MHz real-time counter at the ends
// of the kernel's parts.
#ifdef MI355_PHASE_CLOCKS
__device__ long long band_clocks[6][8];
#define MI355_BAND_PHASE(i)                                   \
    do                                                        \
    {                                                         \
        if (band_row >= 0 && lane == 0)                       \
            band_clocks[band_row][i] = (long long)wall_clock64(); \
    } while (0)
#else
#define MI355_BAND_PHASE(i) \
    do                      \
    {                       \
    } while (0)
#endif

// MULTI: up to NARROW_MAX_PANELS panels of 64 columns (K <= 192, NB == 1), all of them in LDS next to the window: a wave
// takes its 32 pixels through one panel after the other - matrix instructions, then that panel's epilogue - so that the
// window, the arguments and the start of a workgroup are paid once for up to 256 output channels.
// KBU: with several panels, the k blocks of 64 that hold data (K <= 64: 1, <= 128: 2, else 3 - the loop need not cover the
// panel's zeros as it does with one panel, where K is not known when the kernel is built).
template <int EPI, bool FLIP_A, int NB, bool MULTI = false, int KBU = NB * 3>
// (p_Bp, p_ndma: the panel image's address and its size in KiB once more, in front of the argument block. This file is
// compiled with -mllvm -amdgpu-kernarg-preload-count=3: a kernel's first three argument dwords arrive in scalar registers
// with the wave, so the panel's transfers - more than half of all - go out while the block is still being fetched: 10
// scalar loads over 6 cache lines per wave, 0.25 us for the first wave of a workgroup and up to 1 us for the last.)
__global__ __launch_bounds__(HALO_WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void conv_halo_kernel(const int8_t *p_Bp, int32_t p_ndma,
                                                                                                                GemmArgs g)
{
    static_assert(!MULTI || NB == 1, "several panels: one batch of k blocks");
    static_assert(KBU >= 1 && KBU <= NB * 3 && (MULTI || KBU == NB * 3), "k blocks that hold data");
    constexpr int RS = NARROW_ROWS / 16, QS = NARROW_BN / 16;
    constexpr int KBLK  = NB * 3;
    constexpr int PITCH = KBLK * 64 + NARROW_PAD_PIECES * 16;
    constexpr int NPAR  = 1 + QP_COUNT;
    constexpr int NDMA  = KBLK * 4 + NARROW_PAD_PIECES; // transfers of 1 KiB that make up a panel
    // LDS: B panels [npan * 64][PITCH] | par[NPAR][npan * 64], the flag word | (from the next KiB) the staged window
    extern __shared__ __attribute__((aligned(1024))) char smem[];
#define MI355_GLOBAL __attribute__((address_space(1)))
#ifdef MI355_PHASE_CLOCKS
    const long long t_entry = (long long)wall_clock64(); // before the first argument is asked for
#endif
    {
        // ---- the B panels: linear transfers of 1 KiB, wave w those at w, w + HALO_PANEL_WAVES, ... ----
        // Written out with scalar registers of its own choosing: the arguments are in flight here, and temporaries that
        // the compiler places in unused parts of their destination registers make it wait for them first.
        const int      wv = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
        // (The panels start at LDS address 0: this kernel has no static LDS in front of the dynamic area. The address as a
        // value would be one more such temporary.)
        const uint32_t v16 = ((uint32_t)threadIdx.x & 63u) * 16u;
        const uint32_t b_lo = (uint32_t)(uintptr_t)p_Bp, b_hi = (uint32_t)((uintptr_t)p_Bp >> 32);
        if (wv < HALO_PANEL_WAVES && wv < (MULTI ? p_ndma : NDMA)) // (the loop below makes its first pass unasked)
        {
            if constexpr (MULTI)
                asm volatile("s_lshl_b32 s92, %[wv], 10\n\t"
                             "s_mov_b32 s93, %[wv]\n"
                             "1:\n\t"
                             "s_add_u32 s90, %[blo], s92\n\t"
                             "s_addc_u32 s91, %[bhi], 0\n\t"
                             "s_mov_b32 m0, s92\n\t"
                             "global_load_lds_dwordx4 %[v16], s[90:91]\n\t"
                             "s_add_u32 s93, s93, %[step]\n\t"
                             "s_add_u32 s92, s92, %[stepb]\n\t"
                             "s_cmp_lt_i32 s93, %[n]\n\t"
                             "s_cbranch_scc1 1b" ::[wv] "s"(wv),
                             [blo] "s"(b_lo), [bhi] "s"(b_hi), [v16] "v"(v16), [n] "s"(p_ndma),  [step] "i"(HALO_PANEL_WAVES),
                             [stepb] "i"(HALO_PANEL_WAVES * 1024)
                             : "s90", "s91", "s92", "s93", "scc", "memory");
            else
                asm volatile("s_lshl_b32 s92, %[wv], 10\n\t"
                             "s_mov_b32 s93, %[wv]\n"
                             "1:\n\t"
                             "s_add_u32 s90, %[blo], s92\n\t"
                             "s_addc_u32 s91, %[bhi], 0\n\t"
                             "s_mov_b32 m0, s92\n\t"
                             "global_load_lds_dwordx4 %[v16], s[90:91]\n\t"
                             "s_add_u32 s93, s93, %[step]\n\t"
                             "s_add_u32 s92, s92, %[stepb]\n\t"
                             "s_cmp_lt_i32 s93, %[n]\n\t"
                             "s_cbranch_scc1 1b" ::[wv] "s"(wv),
                             [blo] "s"(b_lo), [bhi] "s"(b_hi), [v16] "v"(v16), [n] "i"(NDMA),  [step] "i"(HALO_PANEL_WAVES),
                             [stepb] "i"(HALO_PANEL_WAVES * 1024)
                             : "s90", "s91", "s92", "s93", "scc", "memory");
        }
    }
    ConvGeom  cg = g.conv;
    uintptr_t u_a = (uintptr_t)g.A, u_cv = (uintptr_t)g.epi.colvec, u_qp = (uintptr_t)g.epi.qp, u_fl = (uintptr_t)g.epi.qp_flag;
    int32_t   a_qps = (int32_t)g.epi.qp_stride, wpi = g.tiles_m, rpw = g.tiles_n; // workgroups per image, output rows per workgroup
    uint32_t  magic_wp = g.magic_tiles; // for the division by the staged window's width (see halo_plan)
    uintptr_t u_fill   = (uintptr_t)g.fill16;
    asm volatile("" : "+s"(magic_wp), "+s"(u_fill));
    asm volatile(""
                 : "+s"(cg.H), "+s"(cg.W), "+s"(cg.C), "+s"(cg.KH), "+s"(cg.KW), "+s"(cg.OW), "+s"(cg.OH), "+s"(cg.stride_x),
                   "+s"(cg.stride_y), "+s"(cg.pad_left), "+s"(cg.pad_top), "+s"(cg.dil_x), "+s"(cg.dil_y), "+s"(cg.pad_word),
                   "+s"(cg.magic_C), "+s"(cg.magic_KW), "+s"(cg.magic_OW), "+s"(a_qps), "+s"(u_a), "+s"(u_cv), "+s"(u_qp),
                   "+s"(u_fl), "+s"(wpi), "+s"(rpw));
    const int npan = MULTI ? __builtin_amdgcn_readfirstlane(g.nblocks) : 1, ncols = npan * NARROW_BN; // panels, their columns
    int32_t  *par  = (int32_t *)(smem + ncols * PITCH);
    const MI355_GLOBAL int32_t *const g_colvec = (const MI355_GLOBAL int32_t *)u_cv, *const g_qp = (const MI355_GLOBAL int32_t *)u_qp;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lh = lane >> 4;
#ifdef MI355_PHASE_CLOCKS
    const int band_blk = blockIdx.x == 0 ? 0 : (blockIdx.x == gridDim.x / 2 ? 1 : (blockIdx.x == gridDim.x - 1 ? 2 : -1));
    const int band_row = band_blk < 0 ? -1 : (wave == 0 ? band_blk * 2 : (wave == 12 ? band_blk * 2 + 1 : -1));
#endif
    MI355_BAND_PHASE(0); // arguments fetched
#ifdef MI355_PHASE_CLOCKS
    if (band_row >= 0 && lane == 0)
        band_clocks[band_row][6] = t_entry;
#endif

    // this workgroup's band: output rows [oy0, oy1) of image n. Staged in LDS: the window of input rows and columns
    // under it, padding included - rows iy_first .. iy_first + in_rows - 1, columns -pad_left .. -pad_left + Wp - 1,
    // pixel (r, x) of the window at pixel index r * Wp + x - so that a tap is an address and nothing else
    const int n = (int)blockIdx.x / wpi, part = (int)blockIdx.x - n * wpi;
    const int oy0 = part * rpw, oy1 = min(cg.OH, oy0 + rpw);
    const int P        = (oy1 - oy0) * cg.OW; // output pixels of the band (<= 16 tiles of 32)
    const int Wp       = (cg.OW - 1) * cg.stride_x + (cg.KW - 1) * cg.dil_x + 1;
    const int in_rows  = (oy1 - oy0 - 1) * cg.stride_y + (cg.KH - 1) * cg.dil_y + 1;
    const int iy_first = oy0 * cg.stride_y - cg.pad_top;
    const int staged   = in_rows * Wp;              // pixels
    const int m_base   = (n * cg.OH + oy0) * cg.OW; // GEMM row of the band's first pixel
    // pieces of 16 bytes per pixel and the permutation of a pixel's pieces: piece c of the pixel at LDS pixel index s
    // (counted from the start of LDS: img_off is a multiple of the pixel size) lies at position
    // c ^ (((s >> sw_sh) & sw_m) << 1). With lane l at pixel s + l % 16, piece l / 16 of a block of 4, each of the
    // four batches of 16 lanes a ds_read_b128 is served in (see NARROW_PAD_PIECES) then has its 16 addresses distinct
    // modulo 256 bytes for pixels of 4, 8 and 16 or more pieces (checked by enumeration for every start s).
    const int cpr = cg.C >> 4, lcpr = 31 - __builtin_clz(cpr), lc = lcpr + 4;
    const int sw_m = cpr >= 16 ? 7 : (cpr == 8 ? 3 : 1), sw_sh = cpr >= 16 ? 0 : (cpr == 8 ? 1 : 2);
    // the permutation as a byte offset: ((s << (5 - sw_sh)) & sw_mask) ^ piece * 16, or from the byte offset x = s << lc:
    // ((x >> sw_r) & sw_mask) - the bits of x below the pixel size land below the mask
    const int sw_mask = sw_m << 5, sw_r = lc - (5 - sw_sh);
    const uint32_t lds0    = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;
    const int      img_off = (ncols * PITCH + NPAR * ncols * 4 + 4 + 1023) & ~1023; // (+ 4: the flag word)
    const int      s_img   = img_off >> lc; // LDS pixel index of the window's first pixel

    // epilogue constants (one dword per thread: 6 x 64 of them per panel), the flag word of the requantisation
    // (fetched by the waves that start first - with one panel the threads of waves 0 to 5 hold one constant each, wave 0
    // the flag word - and handed on through LDS: the waves that start last then have nothing to wait for before the barrier)
    const bool    have_qp = EPI == EPI_FIXEDPOINT && u_qp != 0;
    constexpr int TPN     = MULTI ? (NPAR * NARROW_BN * NARROW_MAX_PANELS + HALO_WAVES * 64 - 1) / (HALO_WAVES * 64) : 1;
    int32_t       tp[TPN];
#pragma unroll
    for (int i = 0; i < TPN; ++i)
    {
        tp[i]         = 0;
        const int idx = tid + i * HALO_WAVES * 64;
        if (have_qp && idx < NPAR * ncols)
        {
            const int v = idx / ncols, col = idx - v * ncols;
            tp[i]       = v == 0 ? g_colvec[col] : g_qp[(v - 1) * a_qps + col];
        }
    }
    int qflag = 1;
    if (wave == 0 && have_qp && u_fl != 0)
        qflag = *(const MI355_GLOBAL int32_t *)u_fl;

    // ---- the staged window: transfers of 1 KiB; a lane fetches the piece its LDS position stands for from the image, or
    // 16 bytes of the padding value. (By the first HALO_DMA_WAVES waves only, like the panel's: the later a wave of the
    // workgroup gets its arguments, the less it should have to do before the barrier - the barrier waits for it.) ----
    const int       nimg = ((staged << lc) + 1023) >> 10;
    const uintptr_t img  = u_a + (uintptr_t)((int64_t)n * cg.H * cg.W * cg.C);
    for (int ins = wave; ins < nimg; ins += HALO_DMA_WAVES)
    {
        if (wave >= HALO_DMA_WAVES)
            break;
        {
            const int q = ins * 64 + lane; // position in the window, in pieces
            const int s = q >> lcpr, c = (q & (cpr - 1)) ^ ((((s + s_img) >> sw_sh) & sw_m) << 1);
            const int r = narrow_div(s, magic_wp), x = s - r * Wp;
            const int iy = iy_first + r, ix = x - cg.pad_left;
            // (lanes past the window's end fill LDS nobody looks at)
            const bool      in   = (s < staged) & ((unsigned)iy < (unsigned)cg.H) & ((unsigned)ix < (unsigned)cg.W);
            const uintptr_t from = in ? img + (uint32_t)(((iy * cg.W + ix) << lc) + c * 16) : u_fill;
            narrow_dma16_at((const void *)from, lds0 + (uint32_t)img_off + (uint32_t)ins * 1024u);
        }
    }

    // ---- this wave's tile: 32 consecutive pixels of the band (worked out in front of the barrier by the waves that
    // have to wait there anyway, behind it by the others) ----
    const bool active = wave * NARROW_ROWS < P;
    int32_t    s0[RS]; // LDS byte offset of the top-left tap of each of the tile's rows, plus this lane's 16 bytes of a 64-byte block
    auto       tile_setup = [&]()
    {
#pragma unroll
        for (int rb = 0; rb < RS; ++rb)
        {
            const int lp = min(wave * NARROW_ROWS + rb * 16 + lr, P - 1);
            const int ry = narrow_div(lp, cg.magic_OW), ox = lp - ry * cg.OW;
            s0[rb]       = ((s_img + ry * cg.stride_y * Wp + ox * cg.stride_x) << lc) + lh * 16;
        }
    };
    if (wave < HALO_DMA_WAVES)
        tile_setup();
    MI355_BAND_PHASE(1); // transfers issued, addresses set up
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wave's transfers (and its constant)
    MI355_BAND_PHASE(2); // this wave's transfers have landed
#pragma unroll
    for (int i = 0; i < TPN; ++i)
        if (have_qp && tid + i * HALO_WAVES * 64 < NPAR * ncols)
            par[tid + i * HALO_WAVES * 64] = tp[i];
    if (tid == 0)
        par[NPAR * ncols] = qflag;
    __syncthreads();
    MI355_BAND_PHASE(3); // everybody's transfers have landed
    if (!active)
        return;
    if (wave >= HALO_DMA_WAVES)
        tile_setup();
    const int  qflag_u = __builtin_amdgcn_readfirstlane(par[NPAR * ncols]);
    const bool fast    = have_qp && (qflag_u & 1) == 0;

    // (Different priorities for the waves that share a SIMD - one at a time through the matrix instructions, its epilogue
    // beside the next wave's - paid while the loop carried twice the address arithmetic; with today's loop, equal
    // priorities measured 0.4 us faster on a 8.3 us kernel. Pinning the loop's order with scheduling barriers - all six
    // reads of block kb + 1 in front of the matrix instructions of block kb, where the compiler puts some of the A reads
    // right in front of their first use - measured 0.1 us slower than the compiler's own order.)
    // (One instance of what follows for every wave: a second, for a last tile of 16 pixels or fewer, measured slower -
    // the code is fetched once per workgroup, a path that one wave takes alone pays for its own instruction fetches.)
    auto run_panel = [&](const int pc0) // pc0: the panel's first column
    {
        constexpr int RSX = RS;
        v4i acc[RSX][QS];
#pragma unroll
        for (int i = 0; i < RSX; ++i)
#pragma unroll
            for (int j = 0; j < QS; ++j)
                acc[i][j] = (v4i){0, 0, 0, 0};
        const char *b_rd  = smem + (pc0 + lr) * PITCH + lh * 16;
        const int   nkb   = (g.K + 63) >> 6; // k blocks that hold data (the panel is zero beyond)
        // operand blocks of k block kb: B from the panel, A from the staged window
        auto read_ops = [&](int kb, v4i (&fa)[RSX], v4i (&fb)[QS])
        {
            // (scalar. K may end before the last batch of 3 k blocks does: those blocks meet zeros in the panel and read
            // the first tap again)
            const int kbe = kb < nkb ? kb : 0;
            const int tap = narrow_div(kbe * 64, cg.magic_C), c64 = kbe * 64 - tap * cg.C;
            const int ky = narrow_div(tap, cg.magic_KW), kx = tap - ky * cg.KW;
            const int ds = ((ky * cg.dil_y * Wp + kx * cg.dil_x) << lc) + c64; // the tap and the block within the pixel, in bytes
#pragma unroll
            for (int q = 0; q < QS; ++q)
                fb[q] = *(const v4i *)(b_rd + q * 16 * PITCH + kb * 64);
#pragma unroll
            for (int rb = 0; rb < RSX; ++rb)
            {
                // x: where the piece would lie unpermuted (pixel index << lc, plus the piece's place in the pixel, which
                // stays below the pixel size); the permutation's bits come from the pixel index. Four instructions per
                // read. (All the addresses worked out in front of the loop, or the per-column term as the C operand of a
                // block's first matrix instruction instead of an addition in the epilogue: both measured slower.)
                const int x = s0[rb] + ds;
                fa[rb]      = *(const v4i *)(smem + (x ^ ((x >> sw_r) & sw_mask)));
            }
        };
        v4i fa[2][RSX], fb[2][QS];
        read_ops(0, fa[0], fb[0]);
        // Straight-line code over every k block the panel has (a wave-uniform branch per block made the compiler wait for
        // the operands of the next block before the matrix instructions of this one). K may end before the last batch of 3
        // blocks does: there the panel holds zeros.
#pragma unroll
        for (int kb = 0; kb < KBU; ++kb)
        {
            if (kb + 1 < KBU)
                read_ops(kb + 1, fa[(kb + 1) & 1], fb[(kb + 1) & 1]);
#pragma unroll
            for (int rb = 0; rb < RSX; ++rb)
            {
                v4i a = fa[kb & 1][rb];
                if (FLIP_A)
                    a ^= (int)0x80808080;
#pragma unroll
                for (int q = 0; q < QS; ++q)
                    acc[rb][q] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[kb & 1][q], a, acc[rb][q], 0, 0, 0);
            }
        }
        MI355_BAND_PHASE(4); // matrix instructions issued

        const int row0 = m_base + wave * NARROW_ROWS, a_M = m_base + P; // rows of the GEMM this tile covers, and where the band ends
        if (fast && g.epi.qp_pk16 && (qflag_u & 3) == 0 && g.epi.vec_store && (g.N & 3) == 0)
        {
            // the short form of the requantisation, 4 columns at a time: lane l holds, for row rb * 16 + l % 16, the 4
            // consecutive columns pc0 + q * 16 + 4 * (l / 16) + {0..3}
            const int16_t  o16 = (int16_t)(2 * g.epi.result_offset + 1), lo16 = (int16_t)g.epi.lo, hi16 = (int16_t)g.epi.hi;
            const pk16_t   off2p1 = {o16, o16}, lo = {lo16, lo16}, hi = {hi16, hi16};
            const int32_t *rowvec = g.epi.rowvec;
            const int      a_N    = g.N;
            int32_t        rv[RSX];
            char          *drow[RSX];
#pragma unroll
            for (int rb = 0; rb < RSX; ++rb)
            {
                const int i = row0 + rb * 16 + lr;
                rv[rb]      = (rowvec && i < a_M) ? rowvec[i] : 0;
                drow[rb]    = (char *)g.D + (int64_t)i * g.ldd + pc0 + 4 * lh;
            }
#pragma unroll
            for (int q = 0; q < QS; ++q)
            {
                const int c  = pc0 + q * 16 + 4 * lh;
                const v4i s2 = *(const v4i *)(par + (1 + QP_S2) * ncols + c), r1 = *(const v4i *)(par + (1 + QP_RSM1) * ncols + c);
                const v4i cv = *(const v4i *)(par + c);
                const int32_t s2a[4] = {s2[0], s2[1], s2[2], s2[3]}, r1a[4] = {r1[0], r1[1], r1[2], r1[3]};
#pragma unroll
                for (int rb = 0; rb < RSX; ++rb)
                {
                    int32_t v[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        v[t] = (int32_t)((uint32_t)acc[rb][q][t] + (uint32_t)cv[t] + (uint32_t)rv[rb]);
                    const uint32_t w = std_requant4_pk16(v, s2a, r1a, off2p1, lo, hi);
                    if (row0 + rb * 16 + lr < a_M && c < a_N)
                        *(uint32_t *)(drow[rb] + q * 16) = w;
                }
            }
        }
        else
        {
            // the general forms check rows against g.M: the band's end stands in for it
            GemmArgs gl = g;
            gl.M        = a_M;
            // (the staged constants' form is built for rows of 64 constants: several panels take the general one)
            if constexpr (MULTI)
                epilogue_store_t<EPI, RSX, QS>(acc, gl, row0, pc0, lane, 0);
            else
            {
                if (fast)
                    epilogue_store_fast<RSX, QS, NARROW_BN>(acc, gl, par, row0, 0, 0, lane, 0);
                else
                    epilogue_store_t<EPI, RSX, QS>(acc, gl, row0, 0, lane, 0);
            }
        }
    };
    // (With one panel the call stands alone: as a loop of one iteration - the panel count a compile-time 1 - the compiler laid
    // the same code out differently and config 4 of the benchmark ran 0.5 us slower.)
    if constexpr (MULTI)
    {
        for (int np = 0; np < npan; ++np)
            run_panel(np * NARROW_BN);
    }
    else
        run_panel(0);
    MI355_BAND_PHASE(5); // stores issued
#undef MI355_GLOBAL
}

template <int EPI, bool FLIP_A>
static const void *halo_fn(int nb, bool multi, int K)
{
    if (multi)
    {
        if (nb != 1)
            return nullptr;
        return K <= 64 ? (const void *)conv_halo_kernel<EPI, FLIP_A, 1, true, 1>
                       : (K <= 128 ? (const void *)conv_halo_kernel<EPI, FLIP_A, 1, true, 2> : (const void *)conv_halo_kernel<EPI, FLIP_A, 1, true, 3>);
    }
    switch (nb)
    {
    case 1: return (const void *)conv_halo_kernel<EPI, FLIP_A, 1>;
    case 2: return (const void *)conv_halo_kernel<EPI, FLIP_A, 2>;
    case 3: return (const void *)conv_halo_kernel<EPI, FLIP_A, 3>;
    case 4: return (const void *)conv_halo_kernel<EPI, FLIP_A, 4>;
    case 5: return (const void *)conv_halo_kernel<EPI, FLIP_A, 5>;
    case 6: return (const void *)conv_halo_kernel<EPI, FLIP_A, 6>;
    }
    return nullptr;
}

// The band form for this convolution? Fills rows-per-workgroup / workgroups-per-image / LDS bytes when it applies: more
// tiles of 32 pixels than 4 per compute unit, C a power of two from 64 on, one panel of columns (up to NARROW_MAX_PANELS
// with K <= 192), and a band whose pixels (at most 16 tiles) and input window fit one workgroup; magic_wp: the reciprocal
// (see ConvGeom) of the window's width.
static bool halo_plan(const GemmArgs &a, int epi, int cus, int &rpw, int &wpi, size_t &lds, uint32_t &magic_wp)
{
    const ConvGeom &c = a.conv;
    if (cus <= 0 || (epi != EPI_FIXEDPOINT && epi != EPI_F32) || c.C < 64 || (c.C & (c.C - 1)) != 0 || c.C > 1024)
        return false;
    if (a.N > NARROW_BN && (a.N > NARROW_MAX_PANELS * NARROW_BN || a.K > 192))
        return false;
    const int64_t ncols = (int64_t)((a.N + NARROW_BN - 1) / NARROW_BN) * NARROW_BN;
    const int64_t images = (int64_t)a.M / ((int64_t)c.OH * c.OW);
    if (images * c.OH * c.OW != a.M || (a.M + NARROW_ROWS - 1) / NARROW_ROWS <= (int64_t)NARROW_WAVES * cus)
        return false;
    if (c.OW > HALO_WAVES * NARROW_ROWS)
        return false;
    const int nb = (a.K + 191) / 192;
    // as many workgroups as compute units where the images allow it, bands no longer than 16 tiles
    const int most = HALO_WAVES * NARROW_ROWS / c.OW; // output rows whose pixels fit the 16 waves
    int       parts = (int)std::max<int64_t>(1, ((int64_t)cus + images - 1) / images);
    parts           = std::min(parts, c.OH);
    rpw             = std::min(most, (c.OH + parts - 1) / parts);
    wpi             = (c.OH + rpw - 1) / rpw;
    // the staged window: band + halo + padding (see the kernel)
    const int64_t in_rows = (int64_t)(rpw - 1) * c.stride_y + (int64_t)(c.KH - 1) * c.dil_y + 1;
    const int64_t wp      = (int64_t)(c.OW - 1) * c.stride_x + (int64_t)(c.KW - 1) * c.dil_x + 1;
    const int64_t img_off = (ncols * (nb * 192 + NARROW_PAD_PIECES * 16) + (1 + QP_COUNT) * ncols * 4 + 4 + 1023) & ~(int64_t)1023;
    const int64_t bytes   = img_off + ((in_rows * wp * c.C + 1023) & ~(int64_t)1023);
    if (bytes > 160 * 1024 || images * wpi > (int64_t)INT32_MAX)
        return false;
    magic_wp = wp == 1 ? 0u : (uint32_t)(0x100000000ull / (uint64_t)wp) + 1u; // (pixel indices stay far below 2^32 / wp)
    lds = (size_t)bytes;
    return true;
}

template <int EPI, bool FLIP_A, bool CONV, bool UNI>
static const void *narrow_fn(int nb)
{
    switch (nb)
    {
    case 1: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 1>;
    case 2: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 2>;
    case 3: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 3>;
    case 4: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 4>;
    case 5: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 5>;
    case 6: return (const void *)gemm_narrow_kernel<EPI, FLIP_A, CONV, UNI, 6>;
    }
    return nullptr;
}

template <int EPI>
static const void *narrow_fn_e(bool flip_a, bool conv, bool uni, int nb)
{
    if (conv)
    {
        if (uni)
            return flip_a ? narrow_fn<EPI, true, true, true>(nb) : narrow_fn<EPI, false, true, true>(nb);
        return flip_a ? narrow_fn<EPI, true, true, false>(nb) : narrow_fn<EPI, false, true, false>(nb);
    }
    return flip_a ? narrow_fn<EPI, true, false, false>(nb) : narrow_fn<EPI, false, false, false>(nb);
}

int narrow_panel_chunks(int K)
{
    if (K < 16 || K > NARROW_MAX_NB * 192)
        return 0;
    return (K + 191) / 192 * 12;
}

bool narrow_applies(const GemmArgs &a, bool conv)
{
    if (a.N < 1 || a.N > NARROW_MAX_PANELS * NARROW_BN || a.K < 16 || a.K > NARROW_MAX_NB * 192 || a.K > a.Kp || a.Kp % 64 != 0 || a.M < 1)
        return false;
    if (a.N > NARROW_BN && a.K > 192) // several panels only while the whole patch stays in registers
        return false;
    if (conv)
    {
        // whole 16-byte columns of one tap; the image batch within 31 bits of offset
        const ConvGeom &c = a.conv;
        const int64_t   images = ((int64_t)a.M + (int64_t)c.OH * c.OW - 1) / ((int64_t)c.OH * c.OW);
        return c.C % 16 == 0 && ((uintptr_t)a.A & 15) == 0 && a.K % 16 == 0 && images * c.H * c.W * c.C < ((int64_t)1 << 31);
    }
    // dense: 16-byte aligned rows of whole 16-byte columns, offsets within 31 bits
    return ((uintptr_t)a.A & 15) == 0 && a.lda % 16 == 0 && a.K % 16 == 0 && (int64_t)a.M * a.lda < ((int64_t)1 << 31);
}

int narrow_launch(int epi, bool flip_a, bool conv, const GemmArgs &args, hipStream_t s, bool *band)
{
    if (band)
        *band = false;
    if (!narrow_applies(args, conv) || args.fill16 == nullptr || epi < 0 || epi > 2)
        return (int)hipErrorInvalidValue;
    const int   nb  = (args.K + 191) / 192;
    const bool  uni = conv && args.conv.C % 64 == 0;
    if (conv)
    {
        int      rpw = 0, wpi = 0;
        size_t   hl  = 0;
        uint32_t mwp = 0;
        if (halo_plan(args, epi, device_cus(), rpw, wpi, hl, mwp))
        {
            const int   npan  = (args.N + NARROW_BN - 1) / NARROW_BN;
            const bool  multi = npan > 1;
            const int   K     = args.K;
            const void *hf    = epi == EPI_FIXEDPOINT ? (flip_a ? halo_fn<EPI_FIXEDPOINT, true>(nb, multi, K) : halo_fn<EPI_FIXEDPOINT, false>(nb, multi, K))
                                                      : (flip_a ? halo_fn<EPI_F32, true>(nb, multi, K) : halo_fn<EPI_F32, false>(nb, multi, K));
            if (hf == nullptr)
                return (int)hipErrorInvalidValue;
            static std::atomic<uint32_t> raised_h[2][2][NARROW_MAX_NB + 3];
            std::atomic<uint32_t>       &done = raised_h[epi == EPI_F32 ? 1 : 0][flip_a ? 1 : 0][multi ? NARROW_MAX_NB + (K <= 64 ? 0 : (K <= 128 ? 1 : 2)) : nb - 1];
            int                          dev  = 0;
            if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32)
                return (int)hipErrorInvalidDevice;
            if ((done.load(std::memory_order_acquire) & (1u << dev)) == 0)
            {
                const hipError_t e = hipFuncSetAttribute(hf, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (e != hipSuccess)
                    return (int)e;
                done.fetch_or(1u << dev, std::memory_order_release);
            }
            GemmArgs a = args;
            a.tiles_m = wpi, a.tiles_n = rpw, a.magic_tiles = mwp, a.nblocks = npan;
            const int64_t images = (int64_t)args.M / ((int64_t)args.conv.OH * args.conv.OW);
            int32_t       ndma   = npan * (nb * 12 + NARROW_PAD_PIECES); // KiB of the panel image
            void         *kargs[] = {&a.Bp, &ndma, &a};
            if (band)
                *band = true;
            return (int)hipLaunchKernel(hf, dim3((unsigned)(images * wpi)), dim3(HALO_WAVES * 64), kargs, hl, s);
        }
    }
    const void *fn  = epi == EPI_S32 ? narrow_fn_e<EPI_S32>(flip_a, conv, uni, nb)
                      : epi == EPI_FIXEDPOINT ? narrow_fn_e<EPI_FIXEDPOINT>(flip_a, conv, uni, nb)
                                              : narrow_fn_e<EPI_F32>(flip_a, conv, uni, nb);
    if (fn == nullptr)
        return (int)hipErrorInvalidValue;
    const int    npan = (args.N + NARROW_BN - 1) / NARROW_BN;
    const size_t lds  = (size_t)npan * NARROW_BN * (nb * 192 + NARROW_PAD_PIECES * 16) + (size_t)(1 + QP_COUNT) * npan * NARROW_BN * sizeof(int32_t);
    if (lds > 48 * 1024)
    {
        // once per kernel and device (for the largest panel count the kernel may meet)
        static std::atomic<uint32_t> raised[3][2][2][2][NARROW_MAX_NB];
        std::atomic<uint32_t>       &done = raised[epi][flip_a ? 1 : 0][conv ? 1 : 0][uni ? 1 : 0][nb - 1];
        int                          dev  = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 32)
            return (int)hipErrorInvalidDevice;
        if ((done.load(std::memory_order_acquire) & (1u << dev)) == 0)
        {
            const size_t most = nb == 1 ? (size_t)NARROW_MAX_PANELS * NARROW_BN * (192 + 16 + (1 + QP_COUNT) * sizeof(int32_t)) : lds;
            const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);
            if (e != hipSuccess)
                return (int)e;
            done.fetch_or(1u << dev, std::memory_order_release);
        }
    }
    GemmArgs a = args;
    a.nblocks  = npan;
    // what the A loads' range check compares with
    if (conv)
    {
        const ConvGeom &c      = args.conv;
        const int64_t   images = ((int64_t)args.M + (int64_t)c.OH * c.OW - 1) / ((int64_t)c.OH * c.OW);
        a.a_end                = args.A + images * c.H * c.W * c.C;
    }
    else
        a.a_end = args.A + (int64_t)(args.M - 1) * args.lda + args.K;
    // Workgroups of 4 waves x 32 rows, 4 to a compute unit. When the last round of workgroups would put a fourth
    // workgroup on only a few compute units (they finish last: the kernel's time is theirs), its rows go out in
    // workgroups with fewer working waves, to more compute units.
    const int rows = NARROW_WAVES * NARROW_ROWS;
    const int full = (args.M + rows - 1) / rows, cus = device_cus();
    int       grid = full;
    a.tiles_m = full, a.tiles_n = NARROW_WAVES;
    constexpr int tw = 2; // working waves of a tail workgroup (1 measured the same, 4 is no split: +0.2 us on config 4)
    if (cus > 0 && full > cus && full % cus != 0 && full % cus <= cus / 4 && tw < NARROW_WAVES)
    {
        const int     start     = full - full % cus;
        const int64_t tail_rows = (int64_t)args.M - (int64_t)start * rows;
        a.tiles_m               = start;
        a.tiles_n               = tw;
        grid                    = start + (int)((tail_rows + tw * NARROW_ROWS - 1) / (tw * NARROW_ROWS));
    }
    void *kargs[] = {&a};
    return (int)hipLaunchKernel(fn, dim3(grid), dim3(NARROW_WAVES * 64), kargs, lds, s);
}
} // namespace mi355

#ifdef MI355_PHASE_CLOCKS
// 6 rows (first / middle / last workgroup x wave 0, wave 12) of 8 readings of the 100 MHz counter, of the last launch
extern "C" int mi355_band_clocks_read(long long *out)
{
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(mi355::band_clocks), sizeof(long long) * 48);
}
#endif
