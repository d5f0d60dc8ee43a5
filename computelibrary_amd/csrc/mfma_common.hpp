// Pieces shared by the matrix-core GEMM kernels: LDS swizzle, tile -> workgroup mapping, accumulator epilogue.
#pragma once
#include <type_traits>
#include "internal.hpp"

namespace mi355
{
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// LDS tiles are rows of CPR 16-byte columns. Column c of row r is stored at column c ^ swz(r). The LDS serves a 16-byte
// access 16 lanes (256 bytes, all 64 banks) per clock: 16 consecutive rows reading the same logical column must land in
// 16 different 16-byte bank groups. 16/CPR rows share one 256-byte span, so rows r and r + 16/CPR (same position in the
// span) get different rotations; a staging write (consecutive columns of consecutive rows) is conflict free as well.
template <int CPR>
__device__ __forceinline__ int swz(int row)
{
    return (row / (16 / CPR)) & (CPR - 1);
}

// Tile -> workgroup mapping. Workgroups are handed to the 8 XCDs round-robin and each XCD has its own L2: give every
// XCD a contiguous run of logical tile ids, and walk the tile grid in groups of GM row panels so that a run covers a
// compact GM x (run/GM) patch whose A and B panels are shared inside one L2.
__device__ __forceinline__ void tile_coords(int bid, int nblocks, int tiles_m, int tiles_n, int &tm, int &tn)
{
    int l = bid;
    if ((nblocks & 7) == 0)
        l = (bid & 7) * (nblocks >> 3) + (bid >> 3);
    const int GM      = 4;
    const int per_grp = GM * tiles_n;
    const int grp     = l / per_grp;
    const int first   = grp * GM;
    const int gsize   = min(tiles_m - first, GM);
    const int in_grp  = l - grp * per_grp;
    tm                = first + in_grp % gsize;
    tn                = in_grp / gsize;
}

// The same for a batch of GEMMs launched as one 1-D grid of batch * tiles_m * tiles_n workgroups: the logical ids run
// batch-major, so an XCD's contiguous run covers whole batch entries (their A and B are then fetched into one L2 only).
__device__ __forceinline__ void tile_coords_batched(int bid, int nblocks, int tiles_m, int tiles_n, int &bz, int &tm,
                                                    int &tn)
{
    int l = bid;
    if ((nblocks & 7) == 0)
        l = (bid & 7) * (nblocks >> 3) + (bid >> 3);
    const int tpb = tiles_m * tiles_n;
    bz            = l / tpb;
    l -= bz * tpb;
    const int GM      = 4;
    const int per_grp = GM * tiles_n;
    const int grp     = l / per_grp;
    const int first   = grp * GM;
    const int gsize   = min(tiles_m - first, GM);
    const int in_grp  = l - grp * per_grp;
    tm                = first + in_grp % gsize;
    tn                = in_grp / gsize;
}

// The same map with the two run-time divisors replaced by multiplications with host-computed reciprocals (every wave of
// every block walks this dependent scalar chain before it can do anything else) and the group size, 1 to 4, by shifts.
__device__ __forceinline__ void tile_coords_batched_fast(int bid, int nblocks, int tiles_m, int tiles_n, uint32_t magic_tiles,
                                                         uint32_t magic_group, int &bz, int &tm, int &tn)
{
    int l = bid;
    if ((nblocks & 7) == 0)
        l = (bid & 7) * (nblocks >> 3) + (bid >> 3);
    const int tpb = tiles_m * tiles_n;
    bz            = nblocks == tpb ? 0 : (int)__umulhi((uint32_t)l, magic_tiles);
    l -= bz * tpb;
    const int per_grp = 4 * tiles_n;
    const int grp     = (int)__umulhi((uint32_t)l, magic_group);
    const int first   = grp * 4;
    const int gsize   = min(tiles_m - first, 4);
    const int in_grp  = l - grp * per_grp;
    // in_grp < 4 * tiles_n: x / 3 == (x * 0xAAAB) >> 17 holds for x < 2^16
    tn = gsize == 4 ? in_grp >> 2 : gsize == 2 ? in_grp >> 1 : gsize == 1 ? in_grp : (int)(((uint32_t)in_grp * 0xAAABu) >> 17);
    tm = first + in_grp - tn * gsize;
}

// Row sums of A taken inside the pipelined kernels: a lane holds the 16-byte column lane/16 of row lane%16 of every
// operand block of A it reads; sums[f] collects the bytes of block row f over the whole K loop (sdot4 with ones). The four
// lanes of a row are added up here, the padding the loader flipped along with the data (K steps beyond K hold zeros;
// a flipped zero counts -128) is taken out, and the sum is scaled: sums[f] becomes the per-row term of output row
// f*16 + lane%16, in every lane of that row - the layout the epilogues above take their row terms in.
template <int RS>
__device__ __forceinline__ void finish_row_sums(int32_t (&sums)[RS], int32_t mul, int32_t flipped_pad_bytes)
{
#pragma unroll
    for (int f = 0; f < RS; ++f)
    {
        int32_t v = sums[f];
        v += __shfl_xor(v, 16);
        v += __shfl_xor(v, 32);
        sums[f] = (int32_t)((uint32_t)mul * (uint32_t)(v + 128 * flipped_pad_bytes));
    }
}
__device__ __forceinline__ int32_t sum_bytes(v4i x, int32_t acc)
{
#pragma unroll
    for (int t = 0; t < 4; ++t)
        acc = __builtin_amdgcn_sdot4(x[t], 0x01010101, acc, false);
    return acc;
}

// Accumulator (fm, fn, r) of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32 x 32 block.
// (row0, col0) is the wave's top-left output coordinate.
template <int EPI, int FM, int FN>
__device__ __forceinline__ void epilogue_store(const v16i (&acc)[FM][FN], const GemmArgs &g, int row0, int col0, int lane,
                                               int bz)
{
    const int        lr = lane & 31, lh = lane >> 5;
    const EpiParams &p      = g.epi;
    const int32_t   *colvec = p.colvec + (int64_t)bz * p.colvec_batch_stride;
    const int32_t   *rowvec = p.rowvec ? p.rowvec + (int64_t)bz * p.rowvec_batch_stride : nullptr;
    char            *D      = (char *)g.D;
#pragma unroll
    for (int fn = 0; fn < FN; ++fn)
    {
        const int  j  = col0 + fn * 32 + lr;
        const bool vj = j < g.N;
        int32_t    cv = 0, mu = p.mult_s, sh = p.shift_s;
        float      bf = 0.f;
        if (vj)
        {
            cv = colvec[j];
            if (EPI == EPI_FIXEDPOINT && p.mult)
            {
                mu = p.mult[j];
                sh = p.shift[j];
            }
            if (EPI == EPI_F32 && p.bias_f32)
                bf = p.bias_f32[j];
        }
#pragma unroll
        for (int fm = 0; fm < FM; ++fm)
        {
#pragma unroll
            for (int r = 0; r < 16; ++r)
            {
                const int i = row0 + fm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (vj && i < g.M)
                {
                    const int32_t rv  = rowvec ? rowvec[i] : 0;
                    const int32_t a   = acc[fm][fn][r];
                    const int64_t idx = (int64_t)bz * g.d_batch_stride + (int64_t)i * g.ldd + j;
                    if (EPI == EPI_S32)
                        ((int32_t *)D)[idx] = (int32_t)((uint32_t)a + (uint32_t)cv + (uint32_t)rv +
                                                        (p.accumulate ? (uint32_t)((int32_t *)D)[idx] : 0u));
                    else if (EPI == EPI_FIXEDPOINT)
                        ((int8_t *)D)[idx] = (int8_t)epi_fixedpoint(a, cv, rv, mu, sh, p);
                    else
                        ((float *)D)[idx] = epi_f32(a, (int32_t)((uint32_t)cv + (uint32_t)rv), bf, p.bias_f32 != nullptr,
                                                    p, p.accumulate ? ((float *)D)[idx] : 0.f);
                }
            }
        }
    }
}
// Accumulators of the pipelined kernel: 16 x 16 blocks produced by v_mfma_i32_16x16x64_i8 with the B panel as the first
// matrix operand, i.e. transposed. A wave's sub-tile is RS row slots of 16 rows by QS column slots of 16 columns; lane l
// holds, for every (rs, qs), output row rs*16 + l%16 and the 4 consecutive output columns qs*16 + 4*(l/16) + {0..3}
// in the 4 registers of acc[rs][qs]: per-column parameters are read as 16-byte vectors and 4 results leave in one store.
// (row0, col0) is the wave's top-left output coordinate.
template <int EPI, int RS, int QS>
__device__ __forceinline__ void epilogue_store_t(const v4i (&acc)[RS][QS], const GemmArgs &g, int row0, int col0,
                                                 int lane, int bz, const int32_t *rvk = nullptr, bool use_rvk = false)
{
    const int        lr = lane & 15, lh = lane >> 4;
    const EpiParams &p      = g.epi;
    const int32_t   *colvec = p.colvec + (int64_t)bz * p.colvec_batch_stride;
    const int32_t   *rowvec = p.rowvec ? p.rowvec + (int64_t)bz * p.rowvec_batch_stride : nullptr;
    char            *D      = (char *)g.D;
    int32_t          rv[RS];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
    {
        const int i = row0 + rs * 16 + lr;
        rv[rs]      = use_rvk ? rvk[rs] : ((rowvec && i < g.M) ? rowvec[i] : 0);
    }
#pragma unroll
    for (int qs = 0; qs < QS; ++qs)
    {
        const int j0 = col0 + qs * 16 + 4 * lh; // first of 4 consecutive columns; inside the padded vectors
        const v4i cv = *(const v4i *)(colvec + j0);
        v4i       mu = {p.mult_s, p.mult_s, p.mult_s, p.mult_s};
        v4i       sh = {p.shift_s, p.shift_s, p.shift_s, p.shift_s};
        float     bf[4] = {0.f, 0.f, 0.f, 0.f};
        if (EPI == EPI_FIXEDPOINT && p.mult)
        {
            mu = *(const v4i *)(p.mult + j0);
            sh = *(const v4i *)(p.shift + j0);
        }
        if (EPI == EPI_F32 && p.bias_f32)
        {
#pragma unroll
            for (int t = 0; t < 4; ++t)
                if (j0 + t < g.N)
                    bf[t] = p.bias_f32[j0 + t];
        }
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
        {
            const int i = row0 + rs * 16 + lr;
            if (i >= g.M || j0 >= g.N)
                continue;
            const int64_t idx = (int64_t)bz * g.d_batch_stride + (int64_t)i * g.ldd + j0;
            const bool    vec = p.vec_store && (j0 + 3 < g.N);
            if (EPI == EPI_FIXEDPOINT)
            {
                uint32_t packed = 0;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    packed |= ((uint32_t)epi_fixedpoint(acc[rs][qs][t], cv[t], rv[rs], mu[t], sh[t], p) & 0xFFu) << (8 * t);
                if (vec)
                    *(uint32_t *)(D + idx) = packed;
                else
                {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (j0 + t < g.N)
                            D[idx + t] = (char)(packed >> (8 * t));
                }
            }
            else if (EPI == EPI_S32)
            {
                v4i o, prev = {0, 0, 0, 0};
                if (p.accumulate)
                {
                    if (vec)
                        prev = *(const v4i *)((int32_t *)D + idx);
                    else
                    {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (j0 + t < g.N)
                                prev[t] = ((int32_t *)D)[idx + t];
                    }
                }
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    o[t] = (int32_t)((uint32_t)acc[rs][qs][t] + (uint32_t)cv[t] + (uint32_t)rv[rs] + (uint32_t)prev[t]);
                if (vec)
                    *(v4i *)((int32_t *)D + idx) = o;
                else
                {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (j0 + t < g.N)
                            ((int32_t *)D)[idx + t] = o[t];
                }
            }
            else
            {
                typedef float v4f __attribute__((ext_vector_type(4)));
                v4f o, prev = {0.f, 0.f, 0.f, 0.f};
                if (p.accumulate)
                {
                    if (vec)
                        prev = *(const v4f *)((float *)D + idx);
                    else
                    {
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            if (j0 + t < g.N)
                                prev[t] = ((float *)D)[idx + t];
                    }
                }
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    o[t] = epi_f32(acc[rs][qs][t], (int32_t)((uint32_t)cv[t] + (uint32_t)rv[rs]), bf[t], p.bias_f32 != nullptr, p,
                                   prev[t]);
                if (vec)
                    *(v4f *)((float *)D + idx) = o;
                else
                {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (j0 + t < g.N)
                            ((float *)D)[idx + t] = o[t];
                }
            }
        }
    }
}
// FIXEDPOINT epilogue of the pipelined kernel for multipliers >= 0. The block's per-column constants were staged in LDS
// as par[6][BN]: row 0 the folded offset/bias vector, rows 1..5 the QP_* vectors; col_in_tile is the wave's first
// column inside the block tile. Same accumulator layout as epilogue_store_t.
template <int RS, int QS, int BN>
__device__ __forceinline__ void epilogue_store_fast(const v4i (&acc)[RS][QS], const GemmArgs &g, const int32_t *par,
                                                    int row0, int col0, int col_in_tile, int lane, int bz,
                                                    const int32_t *rvk = nullptr, bool use_rvk = false)
{
    const int        lr = lane & 15, lh = lane >> 4;
    const EpiParams &p      = g.epi;
    const int32_t   *rowvec = p.rowvec ? p.rowvec + (int64_t)bz * p.rowvec_batch_stride : nullptr;
    char            *D      = (char *)g.D;
    int32_t          rv[RS];
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
    {
        const int i = row0 + rs * 16 + lr;
        rv[rs]      = use_rvk ? rvk[rs] : ((rowvec && i < g.M) ? rowvec[i] : 0);
    }
#pragma unroll
    for (int qs = 0; qs < QS; ++qs)
    {
        const int c  = col_in_tile + qs * 16 + 4 * lh;
        const int j0 = col0 + qs * 16 + 4 * lh;
        const v4i cv = *(const v4i *)(par + 0 * BN + c);
        const v4i s2 = *(const v4i *)(par + (1 + QP_S2) * BN + c);
        const v4i cm = *(const v4i *)(par + (1 + QP_CMASK) * BN + c);
        const v4i ls = *(const v4i *)(par + (1 + QP_LS) * BN + c);
        const v4i r1 = *(const v4i *)(par + (1 + QP_RSM1) * BN + c);
        const v4i rm = *(const v4i *)(par + (1 + QP_RMASK) * BN + c);
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
        {
            const int i = row0 + rs * 16 + lr;
            int32_t   o[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
            {
                const int32_t v = (int32_t)((uint32_t)acc[rs][qs][t] + (uint32_t)cv[t] + (uint32_t)rv[rs]);
                o[t]            = fast_requant(v, s2[t], cm[t], ls[t], r1[t], rm[t], p.result_offset, p.lo, p.hi);
            }
            // low bytes of o[0..3] -> one dword
            const uint32_t p01    = __builtin_amdgcn_perm((uint32_t)o[1], (uint32_t)o[0], 0x0c0c0400u);
            const uint32_t p23    = __builtin_amdgcn_perm((uint32_t)o[3], (uint32_t)o[2], 0x0c0c0400u);
            const uint32_t packed = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
            if (i >= g.M || j0 >= g.N)
                continue;
            const int64_t idx = (int64_t)bz * g.d_batch_stride + (int64_t)i * g.ldd + j0;
            if (p.vec_store && (j0 + 3 < g.N))
                *(uint32_t *)(D + idx) = packed;
            else
            {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (j0 + t < g.N)
                        D[idx + t] = (char)(packed >> (8 * t));
            }
        }
    }
}
// The same arithmetic as epilogue_store_fast, but the packed 8-bit results of the whole BM x BN block tile are first
// laid out in LDS (row pitch BN + 16 bytes: the 64 dword writes of a wave instruction - 16 rows by 4 dwords - then hit
// 64 different banks) and then written with 16 bytes per lane, BN/16 lanes per output row, so a wave instruction writes
// whole rows of the tile instead of 16-byte pieces of 16 different rows. All NW consumer waves of the block call this
// together; `barrier` is executed once between the two phases by every wave of the block. Requires p.vec_store16.
// stage must not overlap par. ROWV: a per-row term exists (b_offset != 0) and is added.
template <bool STD, bool ROWV, int RS, int QS, int BM, int BN, int NW, typename Barrier>
__device__ __forceinline__ void epilogue_store_staged(const v4i (&acc)[RS][QS], const GemmArgs &g, const int32_t *par,
                                                      char *stage, int m0, int n0, int row_in_tile, int col_in_tile,
                                                      int wave, int lane, int bz, Barrier barrier,
                                                      const int32_t *rvk = nullptr, bool use_rvk = false)
{
    constexpr int    PITCH = BN + 16;
    const int        lr = lane & 15, lh = lane >> 4;
    const EpiParams &p      = g.epi;
    const int32_t   *rowvec = p.rowvec ? p.rowvec + (int64_t)bz * p.rowvec_batch_stride : nullptr;
    int32_t          rv[RS];
    const int32_t    off2p1 = 2 * p.result_offset + 1;
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
    {
        const int i = m0 + row_in_tile + rs * 16 + lr;
        rv[rs]      = !ROWV ? 0 : (use_rvk ? rvk[rs] : ((rowvec && i < g.M) ? rowvec[i] : 0));
    }
#pragma unroll
    for (int qs = 0; qs < QS; ++qs)
    {
        const int c  = col_in_tile + qs * 16 + 4 * lh;
        const v4i cv = *(const v4i *)(par + 0 * BN + c);
        const v4i s2 = *(const v4i *)(par + (1 + QP_S2) * BN + c);
        const v4i r1 = *(const v4i *)(par + (1 + QP_RSM1) * BN + c);
        v4i       cm = {0, 0, 0, 0}, ls = cm, rm = cm;
        if (!STD)
        {
            cm = *(const v4i *)(par + (1 + QP_CMASK) * BN + c);
            ls = *(const v4i *)(par + (1 + QP_LS) * BN + c);
            rm = *(const v4i *)(par + (1 + QP_RMASK) * BN + c);
        }
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
        {
            int32_t o[4];
#pragma unroll
            for (int t = 0; t < 4; ++t)
            {
                const int32_t v = ROWV ? (int32_t)((uint32_t)acc[rs][qs][t] + (uint32_t)cv[t] + (uint32_t)rv[rs])
                                       : (int32_t)((uint32_t)acc[rs][qs][t] + (uint32_t)cv[t]);
                o[t] = STD ? std_requant(v, s2[t], r1[t], off2p1, p.lo, p.hi)
                           : fast_requant(v, s2[t], cm[t], ls[t], r1[t], rm[t], p.result_offset, p.lo, p.hi);
            }
            const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)o[1], (uint32_t)o[0], 0x0c0c0400u);
            const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)o[3], (uint32_t)o[2], 0x0c0c0400u);
            *(uint32_t *)(stage + (row_in_tile + rs * 16 + lr) * PITCH + c) = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
        }
    }
    barrier();
    constexpr int LPR = BN / 16;  // lanes per output row
    constexpr int RPI = 64 / LPR; // rows per wave instruction
    char         *D   = (char *)g.D + (int64_t)bz * g.d_batch_stride;
    const int     rr = lane / LPR, cc = (lane % LPR) * 16;
#pragma unroll
    for (int it = 0; it < BM / (NW * RPI); ++it)
    {
        const int r = (it * NW + wave) * RPI + rr;
        const int i = m0 + r, j0 = n0 + cc;
        if (i >= g.M || j0 >= g.N)
            continue;
        const v4i     val = *(const v4i *)(stage + r * PITCH + cc);
        const int64_t idx = (int64_t)i * g.ldd + j0;
        if (j0 + 16 <= g.N)
            __builtin_nontemporal_store(val, (v4i *)(D + idx));
        else
        {
            for (int t = 0; t < g.N - j0; ++t)
                D[idx + t] = (char)(val[t >> 2] >> (8 * (t & 3)));
        }
    }
}
// S32 / F32 results of one wave's (RS*16) x (QS*16) sub-tile, 16 rows at a time through a wave-private LDS area
// (16 rows, pitch QS*64 + 16 bytes) so that they leave as 16 bytes per lane along whole row segments of QS*64 bytes
// instead of 16-byte pieces of 16 different rows. Needs no synchronisation with other waves. Requires p.vec_store.
template <int EPI, int RS, int QS>
__device__ __forceinline__ void epilogue_store_wave32(const v4i (&acc)[RS][QS], const GemmArgs &g, char *stage, int row0,
                                                      int col0, int lane, int bz, const int32_t *rvk = nullptr, bool use_rvk = false)
{
    static_assert(EPI == EPI_S32 || EPI == EPI_F32, "32-bit outputs only");
    constexpr int    PITCH = QS * 64 + 16;
    constexpr int    LPR   = QS * 4;   // lanes per output row segment
    constexpr int    RPI   = 64 / LPR; // rows per wave instruction
    static_assert(LPR <= 64 && 16 % RPI == 0, "wave tile width");
    const int        lr = lane & 15, lh = lane >> 4;
    const EpiParams &p      = g.epi;
    const int32_t   *colvec = p.colvec + (int64_t)bz * p.colvec_batch_stride;
    const int32_t   *rowvec = p.rowvec ? p.rowvec + (int64_t)bz * p.rowvec_batch_stride : nullptr;
    char            *D      = (char *)g.D + (int64_t)bz * g.d_batch_stride * 4;
    const int        rr = lane / LPR, cc = lane % LPR;
    // Everything the loop below needs from global memory is fetched before its first store goes out: a wait for a load
    // issued after a store also waits for that store to reach memory, and one such wait per block of 16 x 16 outputs
    // made the epilogue as slow as its slowest store, sixteen times over.
    v4i     cvq[QS];
    float   bfq[QS][4];
    int32_t rvs[RS];
    const bool has_bias = EPI == EPI_F32 && p.bias_f32 != nullptr;
#pragma unroll
    for (int qs = 0; qs < QS; ++qs)
    {
        const int j0 = col0 + qs * 16 + 4 * lh; // inside the padded vectors
        cvq[qs]      = *(const v4i *)(colvec + j0);
#pragma unroll
        for (int t = 0; t < 4; ++t)
            bfq[qs][t] = (has_bias && j0 + t < g.N) ? p.bias_f32[j0 + t] : 0.f;
    }
#pragma unroll
    for (int rs = 0; rs < RS; ++rs)
    {
        const int i = row0 + rs * 16 + lr;
        rvs[rs]     = use_rvk ? rvk[rs] : ((rowvec && i < g.M) ? rowvec[i] : 0);
    }
    // The conditions that are the same for the whole launch (bias, offsets, second clamp) and for the whole tile (inside
    // the matrix or on its edge) are decided once, here, and the loop over the outputs is instantiated for each answer:
    // tested per output they cost about 25 vector instructions each, and with two consumer waves per SIMD that, not the
    // stores, set the length of the epilogue. Inside the matrix a store is a running row pointer and nothing else.
    const bool interior = __builtin_amdgcn_readfirstlane(row0) + RS * 16 <= g.M && __builtin_amdgcn_readfirstlane(col0) + QS * 16 <= g.N;
    auto tile = [&](auto bias_c, auto offs_c, auto twice_c, auto inside_c)
    {
        constexpr bool BIAS = decltype(bias_c)::value, OFFS = decltype(offs_c)::value, TWICE = decltype(twice_c)::value;
        constexpr bool INSIDE = decltype(inside_c)::value;
        char         *dp   = D + ((int64_t)(row0 + rr) * g.ldd + col0 + cc * 4) * 4; // this lane's segment of the first row
        const int64_t step = (int64_t)RPI * g.ldd * 4;
        const float   scale = p.scale, lo = p.act_min, hi = p.act_max;
#pragma unroll
        for (int rs = 0; rs < RS; ++rs)
        {
            const int32_t rv = rvs[rs];
#pragma unroll
            for (int qs = 0; qs < QS; ++qs)
            {
                const v4i cv = cvq[qs];
                v4i       o;
#pragma unroll
                for (int t = 0; t < 4; ++t)
                {
                    const int32_t off = (int32_t)((uint32_t)cv[t] + (uint32_t)rv);
                    if (EPI == EPI_S32)
                        o[t] = (int32_t)((uint32_t)acc[rs][qs][t] + (uint32_t)off);
                    else
                        o[t] = __float_as_int(epi_f32_static<BIAS, OFFS, TWICE>(acc[rs][qs][t], off, bfq[qs][t], scale, lo, hi));
                }
                *(v4i *)(stage + lr * PITCH + (qs * 16 + 4 * lh) * 4) = o;
            }
#pragma unroll
            for (int it = 0; it < 16 / RPI; ++it)
            {
                const int r   = it * RPI + rr;
                const v4i val = *(const v4i *)(stage + r * PITCH + cc * 16);
                if (INSIDE)
                {
                    __builtin_nontemporal_store(val, (v4i *)dp);
                    dp += step;
                    continue;
                }
                const int gi = row0 + rs * 16 + r, j0 = col0 + cc * 4;
                if (gi >= g.M || j0 >= g.N)
                    continue;
                const int64_t idx = ((int64_t)gi * g.ldd + j0) * 4;
                if (j0 + 3 < g.N)
                    __builtin_nontemporal_store(val, (v4i *)(D + idx));
                else
                {
                    for (int t = 0; t < g.N - j0; ++t)
                        *(int32_t *)(D + idx + 4 * t) = val[t];
                }
            }
        }
    };
    using yes = std::true_type;
    using no  = std::false_type;
    auto edge_or_not = [&](auto bias_c, auto offs_c, auto twice_c)
    {
        if (interior)
            tile(bias_c, offs_c, twice_c, yes{});
        else
            tile(bias_c, offs_c, twice_c, no{});
    };
    if (EPI == EPI_S32)
        edge_or_not(no{}, no{}, no{});
    else if (!p.has_offsets)
    {
        if (has_bias)
            edge_or_not(yes{}, no{}, no{});
        else
            edge_or_not(no{}, no{}, no{});
    }
    else if (p.act_twice)
    {
        if (has_bias)
            edge_or_not(yes{}, yes{}, yes{});
        else
            edge_or_not(no{}, yes{}, yes{});
    }
    else
    {
        if (has_bias)
            edge_or_not(yes{}, yes{}, no{});
        else
            edge_or_not(no{}, yes{}, no{});
    }
}
} // namespace mi355
