// Device-side PPE: the integer epilogue every NCE task type runs after accumulation.
// Order of operations follows the reference's register programming
// (src/vpux_compiler/src/dialect/VPUMI37XX/ops/external/runtime_dpu_parser_imports.cpp.inc:511-542
// for PReLU / zero point, :1952-2045 for scale, clamp and rounding registers):
//   x = acc + bias ; x = round_shift(x * mult, shift) ; negative x: x = round_shift(x * prelu_mult,
//   prelu_shift) ; clamp ; + output zero point ; store as u8 / i8.
#pragma once

#include "nce_common.h"

namespace nce {

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

// Full-generality epilogue for one accumulator. Returns the value to store (already in the output
// type's range), as int32.
__device__ __forceinline__ int32_t ppe_apply(int32_t acc, int32_t bias, int32_t mult, int32_t shift,
                                             const PpeDev& p) {
    int64_t x = (int64_t)acc + (int64_t)bias;
    int32_t y = sat_i32(rshift_round(x * (int64_t)mult, shift, p.round_mode));
    if (y < 0 && !(p.prelu_mult == 1 && p.prelu_shift == 0))
        y = sat_i32(rshift_round((int64_t)y * (int64_t)p.prelu_mult, p.prelu_shift, p.round_mode));
    y = y < p.lo ? p.lo : (y > p.hi ? p.hi : y);
    return y + p.zp_out;
}

// Same result as ppe_apply when 1 <= shift, rounding is HALF_UP and |result| cannot leave int32
// (shift >= 17 guarantees it: |x * mult| < 2^48). c = bias * mult + 2^(shift-1) is precomputed per
// output channel so the requantize step is one 64-bit multiply-add and one 64-bit shift.
__device__ __forceinline__ int32_t ppe_apply_fast(int32_t acc, int32_t mult, int32_t shift, int64_t c,
                                                  const PpeDev& p) {
    int32_t y = (int32_t)(((int64_t)acc * (int64_t)mult + c) >> shift);
    if (y < 0 && !(p.prelu_mult == 1 && p.prelu_shift == 0))
        y = sat_i32(rshift_round((int64_t)y * (int64_t)p.prelu_mult, p.prelu_shift, NCE_ROUND_HALF_UP));
    y = y < p.lo ? p.lo : (y > p.hi ? p.hi : y);
    return y + p.zp_out;
}

}  // namespace nce
