// Device-side arithmetic shared by every kernel of the quantized-GEMM path: the fixed-point
// requantisation primitive and the three ways an int32 accumulator leaves the chip.
//
// The integer semantics restate the reference's NEON code:
//   SQDMULH (no rounding) then SRSHL (round half up), src/core/NEON/NEAsymm.h:95-128, :233-296,
//   src/core/NEON/NEMath.inl:430-440; saturating narrow then bounded-relu clamp, NEAsymm.h:130-147.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi355
{
enum : int
{
    EPI_S32        = 0,
    EPI_FIXEDPOINT = 1,
    EPI_F32        = 2
};

struct EpiParams
{
    const int32_t *colvec; // [N]  a_off*colsum[j] + a_off*b_off*K (+ int32 bias[j] for EPI_FIXEDPOINT)
    const int32_t *rowvec; // [M]  b_off*rowsum[i], or nullptr when b_off == 0
    const int32_t *mult;   // [N]  per-channel multipliers, or nullptr (then mult_s)
    const int32_t *shift;  // [N]  per-channel shifts, or nullptr (then shift_s)
    const float   *bias_f32;
    int64_t        colvec_batch_stride; // elements between batches (0: shared B)
    int64_t        rowvec_batch_stride;
    int32_t        mult_s, shift_s;
    int32_t        result_offset;
    int32_t        stage; // 0: QUANTIZE_DOWN_FIXEDPOINT, 1: QUANTIZE_DOWN (integer multiplier, truncating shift)
    int32_t        lo, hi; // clamp range, already intersected with the destination type's range
    float          scale;
    float          act_min, act_max;
    int32_t        has_offsets; // EPI_F32: whether the offset term is added at all
    int32_t        dst_signed;
    int32_t        vec_store; // destination rows / base / batch stride allow 4-element vector stores
    int32_t        vec_store16; // ... and 16-byte stores of 8-bit results
    // Pre-digested per-column requantisation vectors qp[5][qp_stride] (see fast_requant below), or nullptr when some
    // multiplier is negative and the general formula has to be used
    const int32_t *qp;
    int64_t        qp_stride;
    int32_t        qp_std; // |result_offset| < 2^28: std_requant may be used where the flag word allows it
    int32_t        qp_pk16; // ... and |result_offset|, |lo|, |hi| <= 1024: std_requant4_pk16 may be used instead
    // One word written together with qp: 0 when every column has a multiplier >= 2^30 and a shift in [2, 31]
    // (std_requant applies), bit 0 set when some multiplier is negative (then only the general formula applies)
    const int32_t *qp_flag;
    int32_t        accumulate; // EPI_S32 / EPI_F32: add the destination's previous contents (GEMMInfo::accumulate)
    int32_t        act_twice;  // EPI_F32: the activation clamp is also applied before the offset term is added
    // != 0: the pipelined kernels sum the rows of A themselves while its tiles pass through their registers (what
    // compute_row_sums does inside the reference's fused kernels, src/core/NEON/kernels/arm_gemm/quantized.cpp:802-838)
    // and use rowsum_mul * rowsum(A)[i] as the per-row term; rowvec is not read then. Needs K % 16 == 0.
    int32_t        rowsum_mul;
};

// Per-column constants of the branch-free requantisation used by the pipelined kernel's epilogue, valid for
// multipliers >= 0 (everything calculate_quantized_multiplier produces):
//   s2    = (int32)(2*mult mod 2^32), cmask = (2*mult >= 2^31) ? -1 : 0   so that  sqdmulh(a, mult) = mulhi(a, s2) + (a & cmask)
//   ls    = max(-shift, 0)                                              left shift before the multiply
//   rsm1  = max(shift - 1, 0), rmask = shift > 0 ? 1 : 0                 so that  rshr(x) = ((x >> rsm1) + rmask) >> rmask
// Shifts of 32 or more in either direction give 0 in the reference arithmetic: encoded as a zero multiplier.
enum : int
{
    QP_S2 = 0,
    QP_CMASK,
    QP_LS,
    QP_RSM1,
    QP_RMASK,
    QP_COUNT
};

// min(max(x, lo), hi) for lo <= hi as one instruction (the compiler keeps min and max apart: it cannot know lo <= hi)
__device__ __forceinline__ int32_t clamp_med3(int32_t x, int32_t lo, int32_t hi)
{
    int32_t r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(lo), "v"(hi));
    return r;
}

__device__ __forceinline__ int32_t fast_requant(int32_t v, int32_t s2, int32_t cmask, int32_t ls, int32_t rsm1,
                                                int32_t rmask, int32_t result_offset, int32_t lo, int32_t hi)
{
    const int32_t pre = (int32_t)((uint32_t)v << ls);
    const int32_t h   = __mulhi(pre, s2) + (pre & cmask);
    const int32_t r   = ((h >> rsm1) + rmask) >> rmask;
    return clamp_med3((int32_t)((uint32_t)r + (uint32_t)result_offset), lo, hi);
}

// The common case of fast_requant (cmask = -1, ls = 0, rmask = 1, rsm1 >= 1): the rounding increment and the result
// offset are one constant, off2p1 = 2*result_offset + 1, added before the last shift:
// ((x + 1) >> 1) + off == (x + 1 + 2*off) >> 1, and |x| <= 2^30 here, so nothing overflows.
__device__ __forceinline__ int32_t std_requant(int32_t v, int32_t s2, int32_t rsm1, int32_t off2p1, int32_t lo, int32_t hi)
{
    const int32_t h = __mulhi(v, s2) + v;
    return clamp_med3(((h >> rsm1) + off2p1) >> 1, lo, hi);
}

// std_requant of 4 values at once, the 4 results' low bytes packed into one word. After the per-column shift the
// values are narrowed to 16 bits with saturation and the constant, the halving and the clamp work on pairs
// (2.75 vector-ALU slots per value instead of 3.75). Same results as std_requant while |off2p1| <= 2049 and
// -1024 <= lo <= hi <= 1024: a value the narrowing saturates ends beyond +-15359 after the halving and is clamped
// to lo or hi either way.
typedef short pk16_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t std_requant4_pk16(const int32_t (&v)[4], const int32_t (&s2)[4], const int32_t (&rsm1)[4],
                                                      pk16_t off2p1, pk16_t lo, pk16_t hi)
{
    int32_t x[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
        x[t] = (__mulhi(v[t], s2[t]) + v[t]) >> rsm1[t];
    pk16_t a = __builtin_amdgcn_cvt_pk_i16(x[0], x[1]), b = __builtin_amdgcn_cvt_pk_i16(x[2], x[3]);
    a = __builtin_elementwise_add_sat(a, off2p1) >> (pk16_t){1, 1};
    b = __builtin_elementwise_add_sat(b, off2p1) >> (pk16_t){1, 1};
    a = __builtin_elementwise_min(__builtin_elementwise_max(a, lo), hi);
    b = __builtin_elementwise_min(__builtin_elementwise_max(b, lo), hi);
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b), __builtin_bit_cast(uint32_t, a), 0x06040200u);
}

// (a * b * 2) >> 32 with the single saturating case, without 64-bit VALU arithmetic
__device__ __forceinline__ int32_t sqdmulh(int32_t a, int32_t b)
{
    const int32_t  hi = __mulhi(a, b);
    const uint32_t lo = (uint32_t)a * (uint32_t)b;
    const int32_t  r  = (int32_t)(((uint32_t)hi << 1) | (lo >> 31));
    return (a == INT32_MIN && b == INT32_MIN) ? INT32_MAX : r;
}

// (x + 2^(e-1)) >> e without intermediate overflow
__device__ __forceinline__ int32_t rounding_shift_right(int32_t x, int32_t e)
{
    if (e <= 0)
        return x;
    if (e >= 32)
        return 0;
    return (x >> e) + ((x >> (e - 1)) & 1);
}

__device__ __forceinline__ int32_t requant_fixedpoint(int32_t v, int32_t mult, int32_t shift, int32_t result_offset)
{
    int32_t r;
    if (shift < 0)
    {
        const int32_t pre = (-shift >= 32) ? 0 : (int32_t)((uint32_t)v << (-shift));
        r                 = sqdmulh(pre, mult);
    }
    else
    {
        r = rounding_shift_right(sqdmulh(v, mult), shift);
    }
    return (int32_t)((uint32_t)r + (uint32_t)result_offset);
}

// SQRDMULH: (a * b + 2^30) >> 31, saturating the single overflowing case (vqrdmulhq_n_s32, src/core/NEON/NESymm.h:62-69)
__device__ __forceinline__ int32_t sqrdmulh(int32_t a, int32_t b)
{
    if (a == INT32_MIN && b == INT32_MIN)
        return INT32_MAX;
    return (int32_t)(((int64_t)a * (int64_t)b + ((int64_t)1 << 30)) >> 31);
}

// int32 -> QSYMM16 (finalize_quantization_int16, src/core/NEON/NESymm.h:54-85): no result offset; [lo, hi] already
// intersected with the int16 range
__device__ __forceinline__ int32_t requant_fixedpoint_s16(int32_t v, int32_t mult, int32_t shift, int32_t lo, int32_t hi)
{
    int32_t r;
    if (shift < 0)
        r = sqrdmulh((-shift >= 32) ? 0 : (int32_t)((uint32_t)v << (-shift)), mult);
    else
        r = rounding_shift_right(sqrdmulh(v, mult), shift);
    return min(max(r, lo), hi);
}

__device__ __forceinline__ int32_t clamp_i32(int32_t v, int32_t lo, int32_t hi)
{
    return min(max(v, lo), hi);
}

// One element of the FIXEDPOINT epilogue: acc (raw dot product) -> 8-bit value as int32
__device__ __forceinline__ int32_t epi_fixedpoint(int32_t acc, int32_t colv, int32_t rowv, int32_t mult, int32_t shift,
                                                  const EpiParams &p)
{
    const int32_t v = (int32_t)((uint32_t)acc + (uint32_t)colv + (uint32_t)rowv);
    if (p.stage == 1)
    {
        // QUANTIZE_DOWN: offset first, wrap-around multiply, truncating arithmetic shift
        const int32_t r = (int32_t)(((uint32_t)v + (uint32_t)p.result_offset) * (uint32_t)mult) >> (shift & 31);
        return clamp_i32(r, p.lo, p.hi);
    }
    return clamp_i32(requant_fixedpoint(v, mult, shift, p.result_offset), p.lo, p.hi);
}

// float(acc)*scale (+bias) (+ previous destination value) then + float(offset terms)*scale, separate roundings and no
// fused multiply-add, in the order of src/core/NEON/kernels/arm_gemm/quantized.cpp:1000-1017 followed by
// src/cpu/kernels/gemmlowp/generic/neon/fp32.cpp:31-54. The reference clamps twice when an activation the assembly
// GEMM understands is set: inside the dequantising merge (quantized.cpp:1015, before the offset term exists) and again
// as the post-op (src/cpu/operators/CpuGemmLowpMatrixMultiplyCore.cpp:326-332); act_twice reproduces the first one.
__device__ __forceinline__ float epi_f32(int32_t acc, int32_t off, float bias, bool has_bias, const EpiParams &p,
                                         float prev = 0.f)
{
#pragma clang fp contract(off) // the multiply and the add must round separately, as the two NEON instructions do
    float r = (float)acc * p.scale;
    if (has_bias)
        r = r + bias;
    if (p.accumulate)
        r = r + prev;
    if (p.has_offsets)
    {
        if (p.act_twice)
            r = fminf(fmaxf(r, p.act_min), p.act_max);
        const float scaled = (float)off * p.scale;
        r                  = r + scaled;
    }
    return fminf(fmaxf(r, p.act_min), p.act_max);
}
// epi_f32 without accumulation, with the launch-wide conditions as template arguments: a tile's epilogue picks one of the
// instances once instead of testing the flags for every output.
template <bool BIAS, bool OFFS, bool TWICE>
__device__ __forceinline__ float epi_f32_static(int32_t acc, int32_t off, float bias, float scale, float lo, float hi)
{
#pragma clang fp contract(off)
    float r = (float)acc * scale;
    if (BIAS)
        r = r + bias;
    if (OFFS)
    {
        if (TWICE)
            r = fminf(fmaxf(r, lo), hi);
        const float scaled = (float)off * scale;
        r                  = r + scaled;
    }
    return fminf(fmaxf(r, lo), hi);
}
} // namespace mi355
