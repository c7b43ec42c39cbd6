// Device-side PPE: the integer epilogue every NCE task type runs after accumulation.
// Order of operations follows the reference's register programming
// (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:511-542
// for PReLU / zero point, :1952-2045 for scale, clamp and rounding registers):
//   x = acc + bias ; x = round_shift(x * mult, shift) ; saturate to int32 ;
//   negative x: x = round_shift(x * prelu_mult, prelu_shift) ; saturate ; clamp ; + zero point.
//
// Two implementations of the same function:
//   * ppe_apply      - 64-bit integer arithmetic, any shift 0..63.
//   * ppe_apply_f64  - the same value through FP64 (gfx950 issues FP64 FMA and conversions at the 32-bit
//                      rate; a general 64-bit shift-and-round takes several instructions). Exact, not approximate: with
//                      M = mult * 2^-shift and B = bias * M + 1/2, the quantity acc * M + B equals
//                      N / 2^shift for an integer |N| < 2^53 whenever shift <= 52, so one FMA
//                      returns it without rounding and floor() (or rint() for ties-to-even) is the
//                      integer pipeline's rounding shift. The kernels also fold the output zero point
//                      (up to 8 more integer bits: zp * 2^shift joins N) into B, so the limit they use
//                      is shift <= 44; larger shifts take the integer path.
#pragma once

#include "nce_common.h"

namespace nce {

constexpr int kMaxF64Shift = 44;  // largest shift for which the FP64 formulation, zero point folded in, is exact

// Can round_shift((acc + bias) * mult, shift) leave int32 for any |acc| <= acc_bound ?
// (It cannot once shift >= 18, because |x * mult| < 2^48; smaller shifts are fine for small sums.)
__host__ __device__ inline bool ppe_may_saturate(int64_t acc_bound, int32_t bias, int32_t mult, int32_t shift) {
    const int64_t b = acc_bound + (bias < 0 ? -(int64_t)bias : (int64_t)bias);
    return ((b * (int64_t)mult) >> shift) + 1 >= 2147483647LL;
}

__device__ __forceinline__ int64_t rshift_round(int64_t p, int32_t s, int32_t mode) {
    if (s <= 0) return p;
    if (mode == NCE_ROUND_HALF_UP) return (p + ((int64_t)1 << (s - 1))) >> s;
    if (mode == NCE_ROUND_NONE) return p >> s;
    const int64_t q = p >> s;
    const int64_t r = p & (((int64_t)1 << s) - 1);
    const int64_t h = (int64_t)1 << (s - 1);
    return q + (int64_t)((r > h) || (r == h && (q & 1)));
}

__device__ __forceinline__ int32_t sat_i32(int64_t v) {
    return v > 2147483647LL ? 2147483647 : (v < -2147483648LL ? (int32_t)(-2147483647 - 1) : (int32_t)v);
}

// Weight-table word [2], 37XX integer packing: mult in bits 31:16, shift in bits 13:8
// (src/vpux_compiler/src/dialect/VPU/utils/nce_sparsity.cpp:141-155).
__device__ __forceinline__ int32_t table_mult(int32_t w2) {
    return (int32_t)((uint32_t)w2 >> 16);
}
__device__ __forceinline__ int32_t table_shift(int32_t w2) {
    return (int32_t)(((uint32_t)w2 >> 8) & 0x3Fu);
}

// Integer path. Returns the value to store (already in the output type's range).
__device__ __forceinline__ int32_t ppe_apply(int32_t acc, int32_t bias, int32_t mult, int32_t shift,
                                             const PpeDev& p) {
    int64_t x = (int64_t)acc + (int64_t)bias;
    int32_t y = sat_i32(rshift_round(x * (int64_t)mult, shift, p.round_mode));
    if (y < 0 && !(p.prelu_mult == 1 && p.prelu_shift == 0))
        y = sat_i32(rshift_round((int64_t)y * (int64_t)p.prelu_mult, p.prelu_shift, p.round_mode));
    y = y < p.lo ? p.lo : (y > p.hi ? p.hi : y);
    return y + p.zp_out;
}

// ---- FP64 path ------------------------------------------------------------------------------

// Per-channel constants: M = mult * 2^-shift, B = bias * M + (1/2 when rounding half-up and shift > 0).
__device__ __forceinline__ double ppe_scale_M(int32_t mult, int32_t shift) {
    return __builtin_ldexp((double)mult, -shift);
}
__device__ __forceinline__ double ppe_scale_B(int32_t bias, double M, int32_t shift, int32_t round_mode) {
    return __builtin_fma((double)bias, M, (round_mode == NCE_ROUND_HALF_UP && shift > 0) ? 0.5 : 0.0);
}

// Wavefront-uniform part of the FP64 epilogue.
struct PpeF64 {
    double pm, pc;   // PReLU slope as prelu_mult * 2^-prelu_shift and its rounding constant
    int32_t lo, hi, zp;
    int32_t lo_zp, hi_zp;  // clamp bounds with the zero point added (folded mode)
    bool even;       // ties-to-even (rint) instead of floor
    bool round_none; // plain floor
    bool sat;        // the requantized value may leave int32 (see ppe_may_saturate)
    bool prelu;      // slope differs from identity
    bool prelu_sat;  // slope result may leave int32
};

__device__ __forceinline__ PpeF64 ppe_f64_setup(const PpeDev& p, bool may_saturate) {
    PpeF64 u;
    u.pm = __builtin_ldexp((double)p.prelu_mult, -p.prelu_shift);
    u.pc = (p.round_mode == NCE_ROUND_HALF_UP && p.prelu_shift > 0) ? 0.5 : 0.0;
    u.lo = p.lo;
    u.hi = p.hi;
    u.zp = p.zp_out;
    u.lo_zp = p.lo + p.zp_out;
    u.hi_zp = p.hi + p.zp_out;
    u.even = p.round_mode == NCE_ROUND_HALF_EVEN;
    u.round_none = p.round_mode == NCE_ROUND_NONE;
    u.sat = may_saturate;
    u.prelu = !(p.prelu_mult == 1 && p.prelu_shift == 0);
    const int64_t am = p.prelu_mult < 0 ? -(int64_t)p.prelu_mult : (int64_t)p.prelu_mult;
    u.prelu_sat = am > ((int64_t)1 << p.prelu_shift);
    return u;
}

// clamp(y, lo, hi) for lo <= hi. Plain min/max (not inline asm) so that the scheduler stays free to
// interleave the independent per-element chains.
__device__ __forceinline__ int32_t med3_i32(int32_t y, int32_t lo, int32_t hi) {
    return min(max(y, lo), hi);
}

// clamp(y, lo, hi) for lo <= hi as ONE instruction (the compiler cannot prove lo <= hi for run-time bounds and
// would emit max + min).
__device__ __forceinline__ int32_t clamp_med3(int32_t y, int32_t lo, int32_t hi) {
    int32_t r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(y), "v"(lo), "v"(hi));
    return r;
}

__device__ __forceinline__ double clamp_i32_range(double v) {
    return __builtin_fmin(__builtin_fmax(v, -2147483648.0), 2147483647.0);
}

// The wavefront-uniform flags are COMPILE-TIME here: a run-time flag inside the per-element code
// makes the compiler evaluate both sides and select, which triples the instruction count.
// v = acc * M + B already formed by the caller (so that callers can fold more terms into it).
template <bool EVEN, bool SAT, bool PRELU, bool PSAT>
__device__ __forceinline__ int32_t ppe_finish_f64_t(double v, const PpeF64& u) {
    v = EVEN ? __builtin_rint(v) : __builtin_floor(v);
    if (SAT) v = clamp_i32_range(v);
    if (PRELU) {
        double r = __builtin_fma(v, u.pm, u.pc);
        r = EVEN ? __builtin_rint(r) : __builtin_floor(r);
        if (PSAT) r = clamp_i32_range(r);
        v = v < 0.0 ? r : v;
    }
    const int32_t y = (int32_t)v;  // in range by construction
    return med3_i32(y, u.lo, u.hi) + u.zp;
}

// Fastest form: round half-up, no saturation, no slope, and the output zero point already folded into
// B and into the clamp bounds (floor(x + zp) = floor(x) + zp for an integer zp).
__device__ __forceinline__ int32_t ppe_finish_f64_folded(double v, int32_t lo_zp, int32_t hi_zp) {
    return med3_i32((int32_t)__builtin_floor(v), lo_zp, hi_zp);
}

// Which specialisation a workgroup runs (uniform). FOLDED and SLOPE cover rounding half-up without
// int32 saturation (every shift >= 18), with or without a negative slope; every other combination
// (ties-to-even, floor, tiny shifts, slopes that can overflow) runs the integer path.
// (PPE_MODE_HI, PPE_MODE_HI_SLOPE: the folded and slope modes in 64-bit integer arithmetic; a kernel that sets
// up their constants opts in.)
enum { PPE_MODE_FOLDED = 0, PPE_MODE_SLOPE = 1, PPE_MODE_INT = 3, PPE_MODE_HI = 4, PPE_MODE_HI_SLOPE = 5 };

__device__ __forceinline__ int ppe_mode_of(const PpeF64& u, bool use_int) {
    if (use_int || u.even || u.sat || u.round_none) return PPE_MODE_INT;
    if (!u.prelu) return PPE_MODE_FOLDED;
    if (!u.prelu_sat) return PPE_MODE_SLOPE;
    return PPE_MODE_INT;
}

template <int MODE>
__device__ __forceinline__ int32_t ppe_finish_mode(double v, const PpeF64& u) {
    if (MODE == PPE_MODE_FOLDED) return ppe_finish_f64_folded(v, u.lo_zp, u.hi_zp);
    return ppe_finish_f64_t<false, false, true, false>(v, u);
}

// B constant of a channel for the given mode: the folded mode carries the output zero point.
__device__ __forceinline__ double ppe_mode_B(double B, int mode, const PpeF64& u) {
    return mode == PPE_MODE_FOLDED ? B + (double)u.zp : B;
}

}  // namespace nce
