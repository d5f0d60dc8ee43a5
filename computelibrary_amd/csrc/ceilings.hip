// Measurement-only kernels: what the machine reaches on the parts a GEMM kernel is made of, at the shapes the library's
// kernels use them. Built into its own shared library (libmi355ceilings.so) that bench.py --ceilings loads; the product
// library does not link this file and nothing here is on the hot path.
//
//   mi355_ceiling_read        one streaming pass over a buffer (the skinny GEMM's B stream, without any arithmetic)
//   mi355_ceiling_mfma        int8 matrix instructions out of registers only (no LDS, no global traffic)
//   mi355_ceiling_mfma_lds    the same instruction count with every operand read from LDS first (64 x 64 wave tiles),
//                             the plain schedule: all reads of a K step, then its matrix instructions, then a barrier
//   mi355_ceiling_mfma_lds_pipelined   the same with operands double-buffered in registers, reads interleaved with the
//                             matrix instructions, no barrier; 64 x 64, 128 x 64 or 64 x 128 wave tiles, or only A from LDS
//                             and the B operand blocks straight from global memory
//   mi355_ceiling_lds_read    the operand reads of the pipelined GEMM alone (LDS bandwidth per compute unit)
//   mi355_ceiling_dma         the pipelined GEMM's global -> LDS stream alone (direct-to-LDS loads, 3-slot ring)
//   mi355_ceiling_clock       shader clock while other work runs: shader-clock ticks over a span of real time
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace
{
// What one workgroup leaves behind for the host (4 x int64 per workgroup, overwritten by every launch): the earliest
// start and the latest end of its waves' timed loops on the 100 MHz real-time counter, and the longest and the summed
// loop duration in shader clocks. The host takes the minimum start and the maximum end over all workgroups: the span
// in which the chip worked on the loops, which is what a rate has to be computed from - the scheduler favours the
// oldest wave of a SIMD, so the loop of any single wave (the first of its workgroup least of all) says little.
__device__ __forceinline__ void leave_span(int64_t *spans, int64_t r0, int64_t r1, int64_t clocks)
{
    __shared__ int64_t w_r0[16], w_r1[16], w_ck[16];
    const int          wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0)
        w_r0[wave] = r0, w_r1[wave] = r1, w_ck[wave] = clocks;
    __syncthreads();
    if (threadIdx.x == 0 && spans)
    {
        int64_t a = w_r0[0], b = w_r1[0], mx = w_ck[0], sum = w_ck[0];
        for (int w = 1; w < nw; ++w)
        {
            a = w_r0[w] < a ? w_r0[w] : a, b = w_r1[w] > b ? w_r1[w] : b;
            mx = w_ck[w] > mx ? w_ck[w] : mx, sum += w_ck[w];
        }
        int64_t *o = spans + (int64_t)blockIdx.x * 4;
        o[0] = a, o[1] = b, o[2] = mx, o[3] = sum;
    }
}

// PATTERN 0: workgroup b owns the contiguous chunk b of the buffer and its waves split that chunk into contiguous
// slices (what a kernel with one workgroup per group of output columns does). PATTERN 1: the whole grid reads one
// contiguous window per iteration (wave w of the grid takes block it * waves + w), the DRAM-friendliest order.
template <int PATTERN, int UNROLL>
__global__ __launch_bounds__(512) void read_kernel(const v4i *__restrict__ src, int64_t kib, int *sink)
{
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int64_t waves = (int64_t)gridDim.x * nw, gw = (int64_t)blockIdx.x * nw + wave;
    v4i           acc = {0, 0, 0, 0};
    if (PATTERN == 0)
    {
        const int64_t per = kib / waves; // 1 KiB blocks per wave (the host passes a multiple)
        const v4i    *p   = src + gw * per * 64 + lane;
        for (int64_t i = 0; i + UNROLL <= per; i += UNROLL)
        {
            v4i t[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                t[u] = __builtin_nontemporal_load(p + (i + u) * 64);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                acc += t[u];
        }
    }
    else
    {
        for (int64_t blk = gw * UNROLL; blk + UNROLL <= kib; blk += waves * UNROLL)
        {
            v4i t[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                t[u] = __builtin_nontemporal_load(src + (blk + u) * 64 + lane);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                acc += t[u];
        }
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678)
        sink[0] = 1;
}

// SHAPE 16: v_mfma_i32_16x16x64_i8, SHAPE 32: v_mfma_i32_32x32x32_i8 (the same multiply-accumulates per instruction
// pair). Every wave issues `mfma16` instructions' worth of work (counted in 16x16x64 units) on operands it read once.
template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_kernel(const v4i *__restrict__ src, int mfma16, int *sink, int64_t *ticks, int64_t *spans)
{
    extern __shared__ char reserve[]; // (the host asks for more than half of LDS: one workgroup per compute unit)
    const int tid = blockIdx.x * blockDim.x + threadIdx.x;
    v4i       a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        a[i] = src[(tid * 16 + i) & 0xFFFFF];
        b[i] = src[(tid * 16 + 8 + i) & 0xFFFFF];
    }
    const int64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    int           s  = 0;
    if (SHAPE == 32)
    {
        v16i acc[4];
        for (int i = 0; i < 4; ++i)
            for (int r = 0; r < 16; ++r)
                acc[i][r] = 0;
        for (int it = 0; it < mfma16 / 32; ++it)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                acc[i & 3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 7], b[(i * 3) & 7], acc[i & 3], 0, 0, 0);
        for (int i = 0; i < 4; ++i)
            for (int r = 0; r < 16; ++r)
                s += acc[i][r];
    }
    else
    {
        v4i acc[8];
        for (int i = 0; i < 8; ++i)
            acc[i] = (v4i){0, 0, 0, 0};
        for (int it = 0; it < mfma16 / 32; ++it)
#pragma unroll
            for (int i = 0; i < 32; ++i)
                acc[i & 7] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i & 7], b[(i * 3) & 7], acc[i & 7], 0, 0, 0);
        for (int i = 0; i < 8; ++i)
            for (int r = 0; r < 4; ++r)
                s += acc[i][r];
    }
    const int64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    sink[tid] = s;
    if (ticks && threadIdx.x == 0 && blockIdx.x == 100 % gridDim.x)
        ticks[0] = t1 - t0, ticks[1] = r1 - r0;
    leave_span(spans, r0, r1, t1 - t0);
}

// 8 waves per workgroup; per K step of 128 every wave reads the operands of a 64 x 64 wave tile (16 x ds_read_b128)
// from a 48 KiB stage of random bytes and issues 32 matrix instructions; one barrier per step.
__global__ __launch_bounds__(512) void mfma_lds_kernel(const v4i *__restrict__ src, int steps, int *sink, int64_t *ticks, int64_t *spans)
{
    extern __shared__ __attribute__((aligned(1024))) char smem[]; // 3 x 48 KiB
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 3 * 49152 / 16; i += blockDim.x)
        ((v4i *)smem)[i] = src[(blockIdx.x * 9216 + i) & 0xFFFFF];
    __syncthreads();
    v4i acc[16];
    for (int i = 0; i < 16; ++i)
        acc[i] = (v4i){0, 0, 0, 0};
    const int64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int kt = 0; kt < steps; ++kt)
    {
        // rows of 128 bytes; lane -> row lane % 16 of an operand block, 16-byte column (kk * 4 + lane / 16) ^ (row & 7):
        // conflict free. A blocks: wave's 4 of the 16 A row blocks, B blocks: 4 of the 8 B row blocks
        const char *s = smem + (kt % 3) * 49152;
        v4i         fa[2][4], fb[2][4];
        const int   row = lane & 15, lh = lane >> 4;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int f = 0; f < 4; ++f)
            {
                const int ra = ((wave >> 1) * 4 + f) * 16 + row, rb = 256 + ((wave & 1) * 4 + f) * 16 + row;
                fa[kk][f]    = *(const v4i *)(s + ra * 128 + (((kk * 4 + lh) ^ (ra & 7)) << 4));
                fb[kk][f]    = *(const v4i *)(s + rb * 128 + (((kk * 4 + lh) ^ (rb & 7)) << 4));
            }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[kk][j], fa[kk][i], acc[i * 4 + j], 0, 0, 0);
        __syncthreads();
    }
    const int64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    int           sum = 0;
    for (int i = 0; i < 16; ++i)
        sum += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = sum;
    if (ticks && threadIdx.x == 0 && blockIdx.x == 100 % gridDim.x)
        ticks[0] = t1 - t0, ticks[1] = r1 - r0;
    leave_span(spans, r0, r1, t1 - t0);
}

// The matrix instructions of the 256 x 128 x 128 tile with every operand read from LDS first, scheduled as well as this
// file knows how: the stage holds static data, so nothing waits for a producer and there is no barrier; operands are
// double-buffered in registers by halves of a K step (64 of K), and the reads of the next half are interleaved one by
// one behind the first matrix instructions of this half (what the pipelined GEMM's consumer waves do). Wave tiles of
// (RS * 16) x (QS * 16): 64 x 64 (8 waves, 8 reads per 16 matrix instructions), 128 x 64 or 64 x 128 (4 waves, 12 reads per
// 32). Rows of 128 bytes, 16-byte piece p of row r at position p ^ ((r >> 1) & 7): free of bank conflicts.
// BGLOBAL: the B operand blocks do not pass through LDS at all - they come straight from global memory in operand order
// (1 KiB per block, the 64 lanes' 16 bytes one after the other: the layout the streaming kernel's packed B has), fetched
// one half step ahead into registers; only A is read from LDS. Every workgroup walks its own 512 KiB of B (one of 32
// column tiles of config 2), which the L2 holds.
template <int RS, int QS, bool BGLOBAL>
__global__ __launch_bounds__(512) void mfma_lds_pipelined_kernel(const v4i *__restrict__ src, int steps, int *sink, int64_t *spans)
{
    constexpr int WN = 128 / (QS * 16); // waves along the tile's columns; wave -> (wave / WN, wave % WN)
    extern __shared__ __attribute__((aligned(1024))) char smem[]; // 3 x 48 KiB
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 3 * 49152 / 16; i += blockDim.x)
        ((v4i *)smem)[i] = src[(blockIdx.x * 9216 + i) & 0xFFFFF];
    __syncthreads();
    const int row = lane & 15, lh = lane >> 4;
    uint32_t  offa[RS], offb[QS]; // byte offset of this lane's piece of every operand block, first half of a K step
#pragma unroll
    for (int f = 0; f < RS; ++f)
    {
        const int r = ((wave / WN) * RS + f) * 16 + row;
        offa[f]     = (uint32_t)(r * 128 + ((lh ^ ((r >> 1) & 7)) << 4));
    }
#pragma unroll
    for (int f = 0; f < QS; ++f)
    {
        const int r = 256 + ((wave % WN) * QS + f) * 16 + row;
        offb[f]     = (uint32_t)(r * 128 + ((lh ^ ((r >> 1) & 7)) << 4));
    }
    v4i acc[RS][QS];
#pragma unroll
    for (int i = 0; i < RS; ++i)
#pragma unroll
        for (int j = 0; j < QS; ++j)
            acc[i][j] = (v4i){0, 0, 0, 0};
    v4i fa[2][RS], fb[2][QS];
    // (the second half of a K step lies 4 pieces on: position p ^ 4 of the same row)
    auto read_half = [&](const char *stage, int half, v4i (&a)[RS], v4i (&b)[QS])
    {
#pragma unroll
        for (int f = 0; f < QS; ++f)
            b[f] = *(const v4i *)(stage + (offb[f] ^ (uint32_t)(half * 64)));
#pragma unroll
        for (int f = 0; f < RS; ++f)
            a[f] = *(const v4i *)(stage + (offa[f] ^ (uint32_t)(half * 64)));
    };
    auto multiply = [&](const v4i (&a)[RS], const v4i (&b)[QS])
    {
#pragma unroll
        for (int i = 0; i < RS; ++i)
#pragma unroll
            for (int j = 0; j < QS; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b[j], a[i], acc[i][j], 0, 0, 0);
    };
    auto interleave = [&]()
    {
        // one LDS read behind each of the first RS + QS matrix instructions, the rest of them after
#pragma unroll
        for (int i = 0; i < RS + QS; ++i)
        {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, RS * QS - (RS + QS), 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    const int64_t t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    int           extra = 0;
    if constexpr (!BGLOBAL)
    {
        read_half(smem, 0, fa[0], fb[0]);
        for (int kt = 0; kt < steps; ++kt)
        {
            const char *cur = smem + (kt % 3) * 49152, *nxt = smem + ((kt + 1) % 3) * 49152;
            read_half(cur, 1, fa[1], fb[1]);
            multiply(fa[0], fb[0]);
            interleave();
            read_half(nxt, 0, fa[0], fb[0]); // (after the last step: a read nobody uses)
            multiply(fa[1], fb[1]);
            interleave();
        }
        extra = fb[0][0][0];
    }
    else
    {
        // half steps between a B block's load and its use: 1 - two register sets, as many registers as the LDS-fed form
        // (2 needs a third set: 256 registers and 10 of them spilled, at the 8 waves per compute unit of the product)
        constexpr int BDIST = 1;
        // half step i of the walk: blocks ((i * WN + wave % WN) * QS + q) of this workgroup's 512 KiB
        // (src holds 16 MiB = 2^20 pieces: the index is taken modulo that, like the LDS fill above - 33 K steps of the last
        // of the 32 column tiles would otherwise end 16 KiB beyond the buffer)
        const size_t bbase = (size_t)(blockIdx.x & 31) * (512 * 1024 / 16) + lane;
        v4i        gb[BDIST + 1][QS];
        auto       load_b = [&](int i, v4i (&b)[QS])
        {
            const int ii = i < 2 * steps ? i : 0; // (beyond the end: a load nobody uses)
#pragma unroll
            for (int q = 0; q < QS; ++q)
                b[q] = src[(bbase + (size_t)((ii * WN + wave % WN) * QS + q) * 64) & 0xFFFFF];
        };
        auto read_a = [&](const char *stage, int half, v4i (&a)[RS])
        {
#pragma unroll
            for (int f = 0; f < RS; ++f)
                a[f] = *(const v4i *)(stage + (offa[f] ^ (uint32_t)(half * 64)));
        };
        auto half_step = [&](const v4i (&a)[RS], const v4i (&b)[QS])
        {
            // this half's B blocks are the oldest loads in flight: BDIST younger half steps may stay out
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(BDIST * QS) : "memory");
            multiply(a, b);
#pragma unroll
            for (int i = 0; i < RS; ++i)
            {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, RS * QS - RS, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        static_assert(BDIST == 1, "the rotation below is written out for two register sets");
        load_b(0, gb[0]);
        read_a(smem, 0, fa[0]);
        // 6 half steps per trip (3 K steps: the ring of stages comes round)
        for (int i = 0; i < 2 * steps; i += 6)
        {
#pragma unroll
            for (int u = 0; u < 6; ++u)
            {
                const int   h   = i + u; // half step: K step h / 2, half h % 2
                const char *stg = smem + (((h + 1) / 2) % 3) * 49152;
                load_b(h + 1, gb[(u + 1) & 1]);
                read_a(stg, (h + 1) & 1, fa[(u + 1) & 1]);
                half_step(fa[u & 1], gb[u & 1]);
            }
        }
        extra = gb[0][0][0] + gb[1][0][0];
    }
    const int64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    int           sum = fa[0][0][0] + extra;
#pragma unroll
    for (int i = 0; i < RS; ++i)
#pragma unroll
        for (int j = 0; j < QS; ++j)
            sum += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    sink[blockIdx.x * blockDim.x + threadIdx.x] = sum;
    leave_span(spans, r0, r1, t1 - t0);
}

// LDS operand reads alone: `waves` waves per workgroup, each reading the 16 operand blocks of a 64 x 64 wave tile
// (ds_read_b128, 1 KiB per wave instruction, the conflict-free swizzled addresses of the GEMM) per step, nothing else.
__global__ __launch_bounds__(1024) void lds_read_kernel(int steps, int *sink, int64_t *ticks)
{
    extern __shared__ __attribute__((aligned(1024))) char smem[]; // 48 KiB
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 49152 / 16; i += blockDim.x)
        ((v4i *)smem)[i] = (v4i){i, lane, wave, 1};
    __syncthreads();
    const int      row = lane & 15, lh = lane >> 4;
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;
    uint32_t       addr[2][8];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int f = 0; f < 8; ++f)
        {
            const int r = (f < 4 ? ((wave >> 1) & 3) * 64 + f * 16 : 256 + (wave & 1) * 64 + (f - 4) * 16) + row;
            addr[kk][f] = lds0 + (uint32_t)(r * 128 + (((kk * 4 + lh) ^ (r & 7)) << 4));
        }
    v4i           acc = {0, 0, 0, 0};
    const int64_t t0  = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int kt = 0; kt < steps; ++kt)
    {
        v4i f[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
            asm volatile("ds_read_b128 %0, %1" : "=v"(f[i]) : "v"(addr[i >> 3][i & 7]));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc ^= f[i];
    }
    const int64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    sink[blockIdx.x * blockDim.x + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (ticks && threadIdx.x == 0 && blockIdx.x == 100 % gridDim.x)
        ticks[0] = t1 - t0, ticks[1] = r1 - r0;
}

__device__ __forceinline__ void dma16s(const void *sbase, uint32_t voff, uint32_t lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_addr) : "memory");
}

// The 256 x 128 x 128 tile's stream: workgroup (tm, tn) of an 8 x 32 tile grid (XCD-major order as in the GEMM) moves 48
// units of 1 KiB per K step (32 of its A panel, 16 of its B panel) into a 3-slot ring with `blockDim.x / 64` issuing
// waves, two steps in flight, nothing reads the LDS.
__global__ __launch_bounds__(768) void dma_kernel(const char *A, const char *B, int64_t ld, int steps, int tiles_n, int *sink,
                                                  int64_t *ticks)
{
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char *)smem;
    const int      lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int      l    = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int      tm = (l / (4 * tiles_n)) * 4 + (l % (4 * tiles_n)) % 4, tn = (l % (4 * tiles_n)) / 4;
    const char    *a0 = A + (int64_t)tm * 256 * ld, *b0 = B + (int64_t)tn * 128 * ld;
    const uint32_t vo = (uint32_t)((lane >> 3) * ld + (lane & 7) * 16);
    const int64_t  t0 = __builtin_readcyclecounter(), r0 = wall_clock64();
    for (int kt = 0; kt < steps; ++kt)
    {
        const uint32_t base = lds0 + (uint32_t)(kt % 3) * 49152u;
        for (int u = wave; u < 48; u += nw)
            dma16s((u < 32 ? a0 + (int64_t)u * 8 * ld : b0 + (int64_t)(u - 32) * 8 * ld) + kt * 128, vo, base + (uint32_t)u * 1024u);
        // at most two steps of this wave's loads in flight
        if (48 / nw == 12)
            asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        else if (48 / nw == 6)
            asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const int64_t t1 = __builtin_readcyclecounter(), r1 = wall_clock64();
    __syncthreads();
    sink[blockIdx.x * blockDim.x + threadIdx.x] = ((int *)smem)[threadIdx.x];
    if (ticks && threadIdx.x == 0 && blockIdx.x == 100 % gridDim.x)
        ticks[0] = t1 - t0, ticks[1] = r1 - r0;
}

// One wave: waits `delay` ticks of the 100 MHz real-time counter, then reports the shader-clock ticks that pass during the
// next `span` ticks of it. Launched on a second stream next to the work whose clock is to be known.
__global__ void clock_kernel(int64_t delay, int64_t span, int64_t *ticks)
{
    const int64_t start = wall_clock64();
    while (wall_clock64() - start < delay)
        __builtin_amdgcn_s_sleep(32);
    const int64_t r0 = wall_clock64(), t0 = __builtin_readcyclecounter();
    int64_t       r1 = r0;
    while (r1 - r0 < span)
    {
        __builtin_amdgcn_s_sleep(32);
        r1 = wall_clock64();
    }
    const int64_t t1 = __builtin_readcyclecounter();
    if (threadIdx.x == 0)
        ticks[0] = t1 - t0, ticks[1] = r1 - r0;
}
} // namespace

extern "C"
{
// kib: size of the buffer in KiB, a multiple of grid * waves * unroll (pattern 1: of unroll); pattern 0 / 1 (see
// read_kernel); unroll 4 or 8
int mi355_ceiling_read(const void *buf, int64_t kib, int pattern, int grid, int waves, int unroll, int *sink, void *stream)
{
    if (!buf || !sink || grid < 1 || waves < 1 || waves > 8 || (unroll != 4 && unroll != 8) || kib < 1 ||
        kib % (pattern == 0 ? (int64_t)grid * waves * unroll : (int64_t)unroll) != 0)
        return (int)hipErrorInvalidValue;
    const v4i  *p = (const v4i *)buf;
    hipStream_t s = (hipStream_t)stream;
    if (pattern == 0 && unroll == 8)
        hipLaunchKernelGGL((read_kernel<0, 8>), dim3(grid), dim3(waves * 64), 0, s, p, kib, sink);
    else if (pattern == 0)
        hipLaunchKernelGGL((read_kernel<0, 4>), dim3(grid), dim3(waves * 64), 0, s, p, kib, sink);
    else if (unroll == 8)
        hipLaunchKernelGGL((read_kernel<1, 8>), dim3(grid), dim3(waves * 64), 0, s, p, kib, sink);
    else
        hipLaunchKernelGGL((read_kernel<1, 4>), dim3(grid), dim3(waves * 64), 0, s, p, kib, sink);
    return (int)hipGetLastError();
}

// src: 16 MiB of operand bytes; grid workgroups of 8 waves, each wave issuing mfma16 (a multiple of 32) 16x16x64-sized
// instructions; sink: grid * 512 ints; ticks: 2 x int64 (shader-clock ticks, 100 MHz ticks of one wave's loop) or null
// spans: 4 x int64 per workgroup (see leave_span) or null. One workgroup per compute unit (96 KiB of LDS reserved).
int mi355_ceiling_mfma(const void *src, int shape, int grid, int mfma16, int *sink, int64_t *ticks, int64_t *spans, void *stream)
{
    if (!src || !sink || grid < 1 || mfma16 < 32 || mfma16 % 32 != 0 || (shape != 16 && shape != 32))
        return (int)hipErrorInvalidValue;
    hipStream_t   s       = (hipStream_t)stream;
    constexpr int RESERVE = 96 * 1024;
    static bool   raised  = false;
    if (!raised)
    {
        hipError_t e = hipFuncSetAttribute((const void *)mfma_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize, RESERVE);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)mfma_kernel<32>, hipFuncAttributeMaxDynamicSharedMemorySize, RESERVE);
        if (e != hipSuccess)
            return (int)e;
        raised = true;
    }
    if (shape == 16)
        hipLaunchKernelGGL(mfma_kernel<16>, dim3(grid), dim3(512), RESERVE, s, (const v4i *)src, mfma16, sink, ticks, spans);
    else
        hipLaunchKernelGGL(mfma_kernel<32>, dim3(grid), dim3(512), RESERVE, s, (const v4i *)src, mfma16, sink, ticks, spans);
    return (int)hipGetLastError();
}

// The pipelined form (see mfma_lds_pipelined_kernel). tile: 0 = 64 x 64 wave tiles (8 waves), 1 = 128 x 64 (4 waves),
// 2 = 64 x 128 (4 waves), 3 = 128 x 64 with the B operand blocks straight from global memory (src: at least 16 MiB);
// steps: K steps of 128 (with tile 3 a multiple of 3); every workgroup issues steps * 256 * 128 * 128 multiply-accumulates
int mi355_ceiling_mfma_lds_pipelined(const void *src, int grid, int tile, int steps, int *sink, int64_t *spans, void *stream)
{
    if (!src || !sink || grid < 1 || steps < 1 || tile < 0 || tile > 3 || (tile == 3 && steps % 3 != 0))
        return (int)hipErrorInvalidValue;
    const void *fns[4] = {(const void *)mfma_lds_pipelined_kernel<4, 4, false>, (const void *)mfma_lds_pipelined_kernel<8, 4, false>,
                          (const void *)mfma_lds_pipelined_kernel<4, 8, false>, (const void *)mfma_lds_pipelined_kernel<8, 4, true>};
    static bool raised = false;
    if (!raised)
    {
        for (const void *f : fns)
        {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 3 * 49152);
            if (e != hipSuccess)
                return (int)e;
        }
        raised = true;
    }
    const v4i *p       = (const v4i *)src;
    void      *kargs[] = {(void *)&p, (void *)&steps, (void *)&sink, (void *)&spans};
    return (int)hipLaunchKernel(fns[tile], dim3(grid), dim3(tile == 0 ? 512 : 256), kargs, 3 * 49152, (hipStream_t)stream);
}

int mi355_ceiling_mfma_lds(const void *src, int grid, int steps, int *sink, int64_t *ticks, int64_t *spans, void *stream)
{
    if (!src || !sink || grid < 1 || steps < 1)
        return (int)hipErrorInvalidValue;
    static bool raised = false;
    if (!raised)
    {
        hipError_t e = hipFuncSetAttribute((const void *)mfma_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 3 * 49152);
        if (e != hipSuccess)
            return (int)e;
        raised = true;
    }
    hipLaunchKernelGGL(mfma_lds_kernel, dim3(grid), dim3(512), 3 * 49152, (hipStream_t)stream, (const v4i *)src, steps, sink,
                       ticks, spans);
    return (int)hipGetLastError();
}

// A: at least 2048 rows, B: at least 4096 rows of ld bytes (ld >= steps * 128); grid = 256 (8 x 32 tiles); waves 4, 8 or 12
int mi355_ceiling_dma(const void *A, const void *B, int64_t ld, int steps, int waves, int *sink, int64_t *ticks, void *stream)
{
    if (!A || !B || !sink || (waves != 4 && waves != 8 && waves != 12) || steps < 1 || ld < (int64_t)steps * 128 || ld % 16 != 0 ||
        ld * 8 >= ((int64_t)1 << 32))
        return (int)hipErrorInvalidValue;
    static bool raised = false;
    if (!raised)
    {
        hipError_t e = hipFuncSetAttribute((const void *)dma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 3 * 49152);
        if (e != hipSuccess)
            return (int)e;
        raised = true;
    }
    hipLaunchKernelGGL(dma_kernel, dim3(256), dim3(waves * 64), 3 * 49152, (hipStream_t)stream, (const char *)A, (const char *)B, ld,
                       steps, 32, sink, ticks);
    return (int)hipGetLastError();
}

// grid workgroups of `waves` (4, 8, 12 or 16) waves, each wave reading 16 KiB per step; sink: grid * waves * 64 ints
int mi355_ceiling_lds_read(int grid, int waves, int steps, int *sink, int64_t *ticks, void *stream)
{
    if (!sink || grid < 1 || steps < 1 || (waves != 4 && waves != 8 && waves != 12 && waves != 16))
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(lds_read_kernel, dim3(grid), dim3(waves * 64), 49152, (hipStream_t)stream, steps, sink, ticks);
    return (int)hipGetLastError();
}

// delay, span in 100 MHz ticks (10 ns); afterwards ticks[0] / ticks[1] * 100 MHz is the shader clock over the span
int mi355_ceiling_clock(int64_t delay, int64_t span, int64_t *ticks, void *stream)
{
    if (!ticks || delay < 0 || span < 1 || delay + span > 100000000)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(clock_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, delay, span, ticks);
    return (int)hipGetLastError();
}
}
